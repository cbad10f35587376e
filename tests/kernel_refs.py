"""Plain torch versions of every kernel op, with the signatures of `tokenizer_amd.kernels.Ops`.

They serve two purposes: the GPU tests compare each HIP kernel with its function here, and the
CPU tests hand an instance to the engine in place of the kernel library so that the host-side
orchestration (tables, slots, scheduling) can be checked without a GPU.  This is a test double,
not a product path: the package itself has no CPU fallback.
"""
from __future__ import annotations

import torch


class PlainOps:
    """Every op computes in float32 (float64 if asked) and rounds to the output's dtype at the end."""

    def __init__(self, work=torch.float32):
        self.work = work

    def embedding(self, ids, table, out, scale=1.0):
        out.copy_((table[ids.long()].to(self.work) * scale).to(torch.float32))
        return out

    def add_pair_rmsnorm(self, residual, first, second, weight, eps, out, rows=None, store_residual=True):
        pick = (lambda t: t) if rows is None else (lambda t: t[rows.long()])
        x = pick(residual).to(self.work) + (pick(first).to(self.work) + pick(second).to(self.work))
        if store_residual:
            assert rows is None
            residual.copy_(x.to(torch.float32))
            x = residual.to(self.work)
        if weight is not None:
            x = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight.to(self.work)
        out.copy_(x.to(out.dtype))
        return out

    # ------------------------------------------------------------ attention over a cached latent
    def _turn(self, x, positions, rates):
        """Coordinate j < n/2 of the last axis with coordinate j + n/2, by position * rates[j] (float32 angles)."""
        half = x.shape[-1] // 2
        angles = positions.to(torch.float32)[:, None] * rates.to(torch.float32)[None, :]
        cos, sin = angles.cos().to(self.work), angles.sin().to(self.work)
        while cos.dim() < x.dim():
            cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
        a, b = x[..., :half], x[..., half:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)

    def latent_store(self, rows, q_offset, q_rank, q_norm, kv_offset, kv_rank, kv_norm, rot_dim, rates, eps, positions,
                     slots, k_pages, v_pages, latent_q):
        x = rows.to(self.work)
        latent_q.copy_((self._unit(x[:, q_offset:q_offset + q_rank], eps) * q_norm.to(self.work)).to(latent_q.dtype))
        kept = self._unit(x[:, kv_offset:kv_offset + kv_rank], eps) * kv_norm.to(self.work)
        if rot_dim:
            tail = x[:, kv_offset + kv_rank:kv_offset + kv_rank + rot_dim]
            kept = torch.cat([kept, self._turn(tail, positions, rates)], dim=1)
        if slots is None:
            return
        page_size = k_pages.shape[2]
        kept = kept.to(k_pages.dtype)
        for t in range(rows.shape[0]):
            slot = int(slots[t])
            if slot < 0:
                continue
            page, off = divmod(slot, page_size)
            k_pages[page, 0, off, :] = kept[t]
            v_pages[page, 0, :, off] = kept[t]

    def head_linear(self, x, x_offset, x_head_stride, weight, out, out_offset, out_head_stride):
        heads, n, k = weight.shape
        for h in range(heads):
            a = x[:, h * x_head_stride + x_offset:h * x_head_stride + x_offset + k].to(self.work)
            at = h * out_head_stride + out_offset
            out[:, at:at + n] = (a @ weight[h].to(self.work).t()).to(out.dtype)
        return out

    def rotate_tails(self, q, heads, head_width, tail_offset, dims, rates, positions, out, out_head_stride, out_offset):
        x = q.to(self.work).reshape(q.shape[0], heads, head_width)[:, :, tail_offset:tail_offset + dims]
        turned = self._turn(x, positions, rates).to(out.dtype)
        for h in range(heads):
            at = h * out_head_stride + out_offset
            out[:, at:at + dims] = turned[:, h]
        return out

    # ------------------------------------------------------------ delta rule with a decay per key channel
    def short_conv_silu(self, rows, offsets, widths, taps, state, state_offset, cu_q, first_position, state_slots,
                        entry_of_token, out, bias=None):
        w = self.work
        n_taps, channels = taps.shape[1], sum(widths)
        x = torch.cat([rows[:, o:o + n] for o, n in zip(offsets, widths)], dim=1).to(w)
        for e in range(cu_q.numel() - 1):
            lo, hi = int(cu_q[e]), int(cu_q[e + 1])
            if hi <= lo:
                continue
            slot = int(state_slots[e])
            tail = state[slot, state_offset:state_offset + (n_taps - 1) * channels].to(w).reshape(n_taps - 1, channels)
            if int(first_position[e]) == 0:
                tail = torch.zeros_like(tail)
            seen = torch.cat([tail, x[lo:hi]], dim=0)
            y = torch.zeros((hi - lo, channels), dtype=w)
            if bias is not None:
                y = y + bias.to(w)
            for j in range(n_taps):
                y = y + seen[j:j + hi - lo] * taps[:, j].to(w)
            out[lo:hi] = (y * torch.sigmoid(y)).to(out.dtype)
            state[slot, state_offset:state_offset + (n_taps - 1) * channels] = seen[seen.shape[0] - (n_taps - 1):].reshape(-1).to(state.dtype)
        return out

    def selective_scan(self, x, pre, neg_rate, low, b_offset, c_offset, skip, rows, z_offset, state, cu_q,
                       first_position, state_slots, out, channels, n):
        w = self.work
        soft = lambda v: torch.where(v > 30.0, v, torch.log1p(torch.exp(torch.clamp(v, max=30.0))))
        A = neg_rate.to(w)
        for e in range(cu_q.numel() - 1):
            lo, hi = int(cu_q[e]), int(cu_q[e + 1])
            if hi <= lo:
                continue
            slot = int(state_slots[e])
            S = state[slot, :channels * n].to(w).reshape(channels, n)
            if int(first_position[e]) == 0:
                S = torch.zeros_like(S)
            for t in range(lo, hi):
                step, xt = soft(pre[t].to(w)), x[t].to(w)
                B, C = low[t, b_offset:b_offset + n].to(w), low[t, c_offset:c_offset + n].to(w)
                S = torch.exp(step[:, None] * A) * S + (step * xt)[:, None] * B[None, :]
                y = S @ C + skip.to(w) * xt
                z = rows[t, z_offset:z_offset + channels].to(w)
                out[t] = (y * (z * torch.sigmoid(z))).to(out.dtype)
            state[slot, :channels * n] = S.reshape(-1).to(state.dtype)
        return out

    def add_terms_rmsnorm(self, residual, terms, weight, eps, out, rows=None, store_residual=True, weight2=None,
                          eps2=0.0, out2=None):
        pick = (lambda t: t) if rows is None else (lambda t: t[rows.long()])
        x = pick(residual).to(self.work)
        total = None
        for term, factor, scale in terms:
            part = pick(term).to(self.work) * factor
            if scale is not None:
                part = part * scale.to(self.work)
            total = part if total is None else total + part
        if total is not None:
            x = x + total
        if store_residual:
            assert rows is None
            residual.copy_(x.to(torch.float32))
            x = residual.to(self.work)
        unit = lambda e: x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + e)
        out.copy_((x if weight is None else unit(eps) * weight.to(self.work)).to(out.dtype))
        if out2 is not None:
            out2.copy_((unit(eps2) * weight2.to(self.work)).to(out2.dtype))
        return out

    def scale_cap(self, x, scale, cap):
        y = x.to(self.work) * scale
        if cap:
            y = cap * torch.tanh(y / cap)
        x.copy_(y.to(x.dtype))
        return x

    def route_scores(self, logits, correction, n_experts, n_groups, keep_groups, chosen, weights, softmax=False,
                     group_max=False, gate=None):
        top = chosen.shape[1]
        z = logits.to(torch.float32)
        s = torch.softmax(z[:, :n_experts], dim=-1) if softmax else torch.sigmoid(z[:, :n_experts])
        choice = s if correction is None else s + correction.to(torch.float32)
        if n_groups:
            per = n_experts // n_groups
            grouped = choice.reshape(-1, n_groups, per)
            worth = grouped.max(-1).values if group_max else torch.topk(grouped, min(2, per), dim=-1).values.sum(-1)
            best = torch.topk(worth, keep_groups, dim=-1).indices
            allowed = torch.zeros_like(worth, dtype=torch.bool).scatter_(1, best, True)
            choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(choice.shape)
        ids = torch.topk(choice, top, dim=-1).indices
        picked = torch.gather(s, 1, ids)
        chosen.copy_(ids.to(torch.int32))
        weights.copy_(picked / (picked.sum(-1, keepdim=True) + 1e-20))
        if gate is not None:
            gate.copy_(torch.sigmoid(z[:, n_experts]))

    def delta_scan(self, fresh, decay, neg_rate, rows, beta_offset, state, cu_q, first_position, state_slots, out,
                   heads, groups, d, dv, unit_eps):
        w = self.work
        share = heads // groups
        for e in range(cu_q.numel() - 1):
            lo, hi = int(cu_q[e]), int(cu_q[e + 1])
            if hi <= lo:
                continue
            slot = int(state_slots[e])
            S = state[slot, :heads * d * dv].to(w).reshape(heads, d, dv).clone()
            if int(first_position[e]) == 0:
                S = torch.zeros_like(S)
            for t in range(lo, hi):
                q = fresh[t, :groups * d].to(w).reshape(groups, d)
                k = fresh[t, groups * d:2 * groups * d].to(w).reshape(groups, d)
                v = fresh[t, 2 * groups * d:].to(w).reshape(heads, dv)
                q = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * d ** -0.5).repeat_interleave(share, dim=0)
                k = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)).repeat_interleave(share, dim=0)
                beta = torch.sigmoid(rows[t, beta_offset:beta_offset + heads].to(w))
                g = torch.exp(neg_rate.to(w)[:, None] * torch.nn.functional.softplus(decay[t].to(w).reshape(heads, d)))
                S = g[:, :, None] * S
                u = beta[:, None] * (v - torch.einsum("hdv,hd->hv", S, k))
                S = S + k[:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", S, q).reshape(-1).to(out.dtype)
            state[slot, :heads * d * dv] = S.reshape(-1).to(state.dtype)
        return out

    # ------------------------------------------------------------ sigmoid router with groups, ungated experts
    def route_sigmoid(self, logits, correction, n_groups, keep_groups, chosen, weights):
        top = chosen.shape[1]
        s = torch.sigmoid(logits.to(torch.float32))
        choice = s + correction.to(torch.float32)
        if n_groups:
            per = logits.shape[1] // n_groups
            grouped = choice.reshape(-1, n_groups, per)
            worth = torch.topk(grouped, min(2, per), dim=-1).values.sum(-1)
            best = torch.topk(worth, keep_groups, dim=-1).indices
            allowed = torch.zeros_like(worth, dtype=torch.bool).scatter_(1, best, True)
            choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(choice.shape)
        ids = torch.topk(choice, top, dim=-1).indices
        picked = torch.gather(s, 1, ids)
        chosen.copy_(ids.to(torch.int32))
        weights.copy_(picked / (picked.sum(-1, keepdim=True) + 1e-20))

    def expert_act(self, up, chosen, weights, n_experts, inner, out):
        n_tokens = up.shape[0]
        x = torch.relu(up.to(self.work)).pow(2).reshape(n_tokens, n_experts, inner)
        factor = torch.zeros((n_tokens, n_experts), dtype=self.work)
        factor.scatter_(1, chosen.long(), weights.to(self.work))
        out.zero_()
        out[:, :n_experts * inner] = (factor[:, :, None] * x).reshape(n_tokens, -1).to(out.dtype)
        return out

    def relu2(self, x, out):
        out.copy_(torch.relu(x.to(self.work)).pow(2).to(out.dtype))
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, out, rows=None, store_residual=True):
        x = residual if rows is None else residual[rows.long()]
        x = x.to(self.work)
        if delta is not None:
            d = delta if rows is None else delta[rows.long()]
            x = x + d.to(self.work)
        if store_residual:
            assert rows is None
            residual.copy_(x.to(torch.float32))
            x = residual.to(self.work)
        y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight.to(self.work)
        out.copy_(y.to(out.dtype))
        return out

    def silu_gate(self, gate_up, out, act=None):
        inner = gate_up.shape[1] // 2
        g, u = gate_up[:, :inner].to(self.work), gate_up[:, inner:].to(self.work)
        if act is None:
            out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))
        elif act == "gelu_tanh":
            out.copy_((0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g))) * u).to(out.dtype))
        else:
            alpha, limit, shift = act
            g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
            out.copy_((g * torch.sigmoid(alpha * g) * (u + shift)).to(out.dtype))
        return out

    # ------------------------------------------------------------ several residual streams
    def embedding_streams(self, ids, table, positions, rates, out):
        x = table[ids.long()].to(torch.float32)
        if rates is not None:
            angles = positions.to(torch.float32)[:, None] * rates[None, :]
            x = x.clone()
            x[:, 0::2] += torch.sin(angles)
            x[:, 1::2] += torch.cos(angles)
        out.copy_(x[:, None, :].expand_as(out))
        return out

    def streams_step(self, streams, write, read, gain, eps, out, rows=None, shift=None):
        x = streams.to(self.work)
        if write is not None:
            y = write.y.to(self.work)
            if write.scale is not None:
                y = y * write.scale.to(self.work)
            x = torch.einsum("tsw,sr->trw", x, write.mix.to(self.work)) + write.out.to(self.work)[None, :, None] * y[:, None, :]
            if rows is None:
                streams.copy_(x.to(torch.float32))
                x = streams.to(self.work)
        if rows is not None:
            x = x[rows.long()]
        u = torch.einsum("tsw,s->tw", x, read.to(self.work))
        h = u / torch.sqrt((u * u).mean(dim=-1, keepdim=True) + eps) * gain.to(self.work)
        if shift is not None:
            mu, state, ctx = shift
            h32 = h.to(torch.float32)
            shifted = torch.empty_like(h32)
            self.token_shift(h32, mu, state, ctx.cu_q, ctx.first_position, ctx.state_slots, ctx.entry_of_token, shifted)
            h = shifted
        out.copy_(h.to(out.dtype))
        return out

    fuses_single_shift = True

    def token_shift(self, h, mu, state, cu_q, first_position, state_slots, entry_of_token, out):
        out.copy_(h.to(out.dtype))
        for e in range(cu_q.numel() - 1):
            lo, hi = int(cu_q[e]), int(cu_q[e + 1])
            if hi <= lo:
                continue
            slot = int(state_slots[e])
            before = torch.zeros_like(h[0]) if int(first_position[e]) == 0 else state[slot].clone()
            rows = torch.cat([before[None], h[lo:hi - 1]], dim=0).to(self.work)
            own = h[lo:hi].to(self.work)
            out[lo:hi] = (own + (rows - own) * mu.to(self.work)).to(out.dtype)
            state[slot] = h[hi - 1]
        return out

    # ------------------------------------------------------------------ matrix memory
    def mlstm_scan(self, qkvg, gates, state, cu_q, first_position, state_slots, out, heads, d, dv, cap):
        w = self.work
        size_c, size_n = heads * d * dv, heads * d
        for e in range(cu_q.numel() - 1):
            lo, hi = int(cu_q[e]), int(cu_q[e + 1])
            if hi <= lo:
                continue
            slot = int(state_slots[e])
            row = state[slot].to(w)
            if int(first_position[e]) == 0:
                row = torch.zeros_like(row)
            c = row[:size_c].reshape(heads, d, dv).clone()
            n = row[size_c:size_c + size_n].reshape(heads, d).clone()
            m = row[size_c + size_n:size_c + size_n + heads].clone()
            for t in range(lo, hi):
                q = qkvg[t, :heads * d].to(w).reshape(heads, d) * d ** -0.5
                k = qkvg[t, heads * d:2 * heads * d].to(w).reshape(heads, d)
                v = qkvg[t, 2 * heads * d:2 * heads * d + heads * dv].to(w).reshape(heads, dv)
                i = cap * torch.tanh(gates[t, :heads].to(w) / cap)
                f = torch.nn.functional.logsigmoid(cap * torch.tanh(gates[t, heads:2 * heads].to(w) / cap))
                new_m = torch.maximum(f + m, i)
                keep, take = torch.exp(f + m - new_m), torch.exp(i - new_m)
                c = keep[:, None, None] * c + take[:, None, None] * k[:, :, None] * v[:, None, :]
                n = keep[:, None] * n + take[:, None] * k
                m = new_m
                floor = torch.maximum((n * q).sum(-1).abs(), torch.exp(-m)) + 1e-6
                out[t] = (torch.einsum("hdv,hd->hv", c, q) / floor[:, None]).reshape(-1).to(out.dtype)
            state[slot, :size_c + size_n + heads] = torch.cat([c.reshape(-1), n.reshape(-1), m]).to(state.dtype)
        return out

    def head_norm_gate(self, read, weight, gate_rows, gate_offset, eps, heads, dv, out):
        w = self.work
        o = read.to(w).reshape(-1, heads, dv)
        o = o / torch.sqrt((o * o).mean(dim=-1, keepdim=True) + eps)
        gate = gate_rows[:, gate_offset:gate_offset + heads * dv].to(w)
        out.copy_((o.reshape(-1, heads * dv) * weight.to(w) * torch.sigmoid(gate)).to(out.dtype))
        return out

    def rope_store(self, qkv, bias, positions, cos_sin, slots, k_pages, v_pages, n_q, n_kv, head_dim, value_dim=None):
        if value_dim is not None and value_dim != head_dim:
            return self._store_uneven(qkv, bias, positions, cos_sin, slots, k_pages, v_pages, n_q, n_kv, head_dim, value_dim)
        n_tokens = qkv.shape[0]
        x = qkv.to(self.work)
        if bias is not None:
            x = x + bias.to(self.work)
        x = x.reshape(n_tokens, n_q + 2 * n_kv, head_dim).clone()
        if cos_sin is not None:
            half = head_dim // 2
            cs = cos_sin[positions.long()].to(self.work)
            cos, sin = cs[:, None, :half], cs[:, None, half:]
            rot = x[:, :n_q + n_kv]
            x1, x2 = rot[..., :half], rot[..., half:]
            x[:, :n_q + n_kv] = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
        qkv.copy_(x.reshape(n_tokens, -1).to(qkv.dtype))
        if slots is not None:
            page_size = k_pages.shape[2]
            stored = qkv.reshape(n_tokens, n_q + 2 * n_kv, head_dim)
            for t in range(n_tokens):
                slot = int(slots[t])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_pages[page, :, off, :] = stored[t, n_q:n_q + n_kv]
                v_pages[page, :, :, off] = stored[t, n_q + n_kv:]       # values lie transposed in a page

    def _store_uneven(self, qkv, bias, positions, cos_sin, slots, k_pages, v_pages, n_q, n_kv, d, dv):
        """Value heads of another size than the key heads: rows are [n_q d | n_kv d | n_kv dv]."""
        n_tokens = qkv.shape[0]
        x = qkv.to(self.work)
        if bias is not None:
            x = x + bias.to(self.work)
        rot = x[:, :(n_q + n_kv) * d].reshape(n_tokens, n_q + n_kv, d).clone()
        if cos_sin is not None:
            half = d // 2
            cs = cos_sin[positions.long()].to(self.work)
            cos, sin = cs[:, None, :half], cs[:, None, half:]
            x1, x2 = rot[..., :half], rot[..., half:]
            rot = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
        x = torch.cat([rot.reshape(n_tokens, -1), x[:, (n_q + n_kv) * d:]], dim=1)
        qkv.copy_(x.to(qkv.dtype))
        if slots is not None:
            page_size = k_pages.shape[2]
            keys = qkv[:, n_q * d:(n_q + n_kv) * d].reshape(n_tokens, n_kv, d)
            values = qkv[:, (n_q + n_kv) * d:].reshape(n_tokens, n_kv, dv)
            for t in range(n_tokens):
                slot = int(slots[t])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_pages[page, :, off, :] = keys[t]
                v_pages[page, :, :, off] = values[t]

    def paged_attention(self, qkv, out, k_pages, v_pages, positions, entry_of_token, block_table,
                        n_q, n_kv, head_dim, window, scale, max_position=None, batch=None,
                        value_dim=None, chunk=None, slopes=None, sinks=None, keep_first=0, value_heads=None, softcap=None):
        page_size = k_pages.shape[2]
        group = n_q // n_kv
        share = 1 if value_heads is None else n_kv // value_heads     # key heads that read one value head
        for t in range(qkv.shape[0]):
            if int(entry_of_token[t]) < 0:                   # a token that only fills the batch up
                continue
            pos = int(positions[t])
            table = block_table[int(entry_of_token[t])]
            lo = max(0, pos - window) if window is not None else 0
            if chunk is not None:
                lo = max(lo, pos // chunk * chunk)
            keys = list(range(0, min(keep_first, lo))) + list(range(lo, pos + 1))
            pages = [int(table[j // page_size]) for j in keys]
            assert all(p >= 0 for p in pages), "attention reads a page that was given back"
            offs = [j % page_size for j in keys]
            k = k_pages[pages, :, offs, :].to(self.work)     # [keys, n_kv, d]
            v = v_pages[pages, :, :, offs].to(self.work)      # [keys, n_kv, d]
            q = qkv[t, :n_q * head_dim].reshape(n_q, head_dim).to(self.work)
            k = k.repeat_interleave(group, dim=1)            # [keys, n_q, d]
            v = v.repeat_interleave(group * share, dim=1)
            scores = torch.einsum("hd,khd->hk", q, k) * scale
            if slopes is not None:
                distance = pos - torch.tensor(keys, dtype=self.work)
                scores = scores - slopes.to(self.work)[:, None] * distance[None, :]
            if softcap:
                scores = softcap * torch.tanh(scores / softcap)
            if sinks is None:
                probs = torch.softmax(scores, dim=-1)
            else:
                top = torch.maximum(scores.max(dim=-1).values, sinks.to(self.work))
                e = torch.exp(scores - top[:, None])
                probs = e / (e.sum(dim=-1) + torch.exp(sinks.to(self.work) - top))[:, None]
            out[t] = torch.einsum("hk,khd->hd", probs, v).reshape(-1).to(out.dtype)
        return out

    # ------------------------------------------------------------ norms behind sub-layers, partial rotation, routing
    def _unit(self, x, eps):
        return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)

    def norm_add_rmsnorm(self, residual, delta, post_weight, post_eps, weight, eps, out, rows=None, store_residual=True):
        x = (residual if rows is None else residual[rows.long()]).to(self.work)
        if delta is not None:
            d = (delta if rows is None else delta[rows.long()]).to(self.work)
            if post_weight is not None:
                d = self._unit(d, post_eps) * post_weight.to(self.work)
            x = x + d
        if store_residual and delta is not None:
            assert rows is None
            residual.copy_(x.to(torch.float32))
            x = residual.to(self.work)
        if weight is not None:
            x = self._unit(x, eps) * weight.to(self.work)
        out.copy_(x.to(out.dtype))
        return out

    def norm_rotate_store(self, qkv, bias, positions, rates, dims, slots, k_pages, v_pages, n_q, n_k, n_v, d, dv,
                          q_norm=None, k_norm=None, eps=0.0):
        n_tokens = qkv.shape[0]
        used = (n_q + n_k) * d + n_v * dv
        x = qkv[:, :used].to(self.work)
        if bias is not None:
            x = x + bias[:used].to(self.work)
        q, k, v = x[:, :n_q * d], x[:, n_q * d:(n_q + n_k) * d], x[:, (n_q + n_k) * d:]
        if q_norm is not None:
            q = self._unit(q, eps) * q_norm.to(self.work)
        if k_norm is not None and n_k:
            k = self._unit(k, eps) * k_norm.to(self.work)
        turn = torch.cat([q, k], dim=1).reshape(n_tokens, n_q + n_k, d).clone()
        half = dims // 2
        if half:
            angles = positions.to(torch.float32)[:, None] * rates.to(torch.float32)[None, :]      # float32 angles
            cos, sin = angles.cos().to(self.work)[:, None, :], angles.sin().to(self.work)[:, None, :]
            a, b = turn[..., :half].clone(), turn[..., half:dims].clone()
            turn[..., :half] = a * cos - b * sin
            turn[..., half:dims] = b * cos + a * sin
        qkv[:, :used] = torch.cat([turn.reshape(n_tokens, -1), v], dim=1).to(qkv.dtype)
        if slots is not None:
            page_size = k_pages.shape[2]
            keys = qkv[:, n_q * d:(n_q + n_k) * d].reshape(n_tokens, n_k, d)
            values = qkv[:, (n_q + n_k) * d:used].reshape(n_tokens, n_v, dv)
            for t in range(n_tokens):
                slot = int(slots[t])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_pages[page, :, off, :] = keys[t]
                v_pages[page, :, :, off] = values[t]

    def differential_heads(self, mixed, lam, eps, out_scale, n_heads, group, dv, out):
        n_tokens = mixed.shape[0]
        maps = mixed.to(self.work).reshape(n_tokens, n_heads // group, 2, group, dv)
        o = maps[:, :, 0] - lam.to(self.work).reshape(()) * maps[:, :, 1]            # [T, kv heads, group, dv]
        out.copy_((self._unit(o, eps) * out_scale).reshape(n_tokens, n_heads * dv).to(out.dtype))
        return out

    def sigmoid_head_gate(self, mixed, rows, offset, n_heads, dv):
        gate = torch.sigmoid(rows[:, offset:offset + n_heads].to(self.work))
        x = mixed.to(self.work).reshape(mixed.shape[0], n_heads, dv) * gate[:, :, None]
        mixed.copy_(x.reshape(mixed.shape).to(mixed.dtype))
        return mixed

    def side_gate(self, gate, table, token_ids, offset, dim, out):
        g = gate.to(self.work)
        act = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g)))
        e = torch.zeros_like(act)
        e[:, :dim] = table[token_ids.long()][:, offset:offset + dim].to(self.work)
        out.copy_((act * e).to(out.dtype))
        return out

    def route_top(self, logits, chosen, weights):
        top = chosen.shape[1]
        values, ids = torch.topk(logits.to(torch.float32), top, dim=-1)
        chosen.copy_(ids.to(torch.int32))
        weights.copy_(torch.softmax(values, dim=-1))

    def expert_gate(self, gate_up, chosen, weights, n_experts, inner, shared, out, shared_weight=None):
        n_tokens = gate_up.shape[0]
        x = gate_up.to(self.work)
        out.zero_()
        routed = x[:, :n_experts * 2 * inner].reshape(n_tokens, n_experts, 2, inner)
        factor = torch.zeros((n_tokens, n_experts), dtype=self.work)
        factor.scatter_(1, chosen.long(), weights.to(self.work))
        g, u = routed[:, :, 0], routed[:, :, 1]
        out[:, :n_experts * inner] = (factor[:, :, None] * (g * torch.sigmoid(g) * u)).reshape(n_tokens, -1).to(out.dtype)
        if shared:
            g, u = x[:, n_experts * 2 * inner:n_experts * 2 * inner + shared], x[:, n_experts * 2 * inner + shared:]
            both = g * torch.sigmoid(g) * u
            if shared_weight is not None:
                both = both * shared_weight.to(self.work)[:, None]
            out[:, n_experts * inner:n_experts * inner + shared] = both.to(out.dtype)
        return out

    def linear(self, x, weight, bias=None, out=None, out_dtype=None):
        y = x.to(self.work) @ weight.to(self.work).t()
        if bias is not None:
            y = y + bias.to(self.work)
        if out_dtype is None:
            out_dtype = x.dtype if out is None else out.dtype
        y = y.to(out_dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear_silu_gate(self, x, weight, out=None, act=None):
        inner = weight.shape[0] // 2
        result = torch.empty((x.shape[0], inner), dtype=x.dtype, device=x.device) if out is None else out
        return self.silu_gate(self.linear(x, weight), result, act=act)

    # The fused decode products, as compositions of the ops above.
    fuse_rows = 16

    def can_fuse_decode(self, rows, dtype, hidden=0):
        return 0 < rows <= self.fuse_rows

    def can_rope_store(self, rows, dtype, weight_elements=0):
        return self.fuse_rows < rows <= 64

    def fold_norm(self, hidden):
        return hidden <= 80          # so that the CPU tests of the engine take both routes

    def fused_norm_qkv_rope(self, residual, norm_weight, eps, weight, bias, positions, cos_sin, slots,
                            k_pages, v_pages, n_q, n_kv, head_dim):
        if norm_weight is None:                                  # the rows are normalised already
            x = residual
        else:
            x = torch.empty(residual.shape, dtype=weight.dtype, device=residual.device)
            self.add_rmsnorm(residual.clone(), None, norm_weight, eps, x)
        qkv = (x.to(self.work) @ weight.to(self.work).t())
        if bias is not None:
            qkv = qkv + bias.to(self.work)
        # The fused kernel rotates the float accumulators and rounds once.
        holder = qkv.to(self.work).clone()
        work_k = None if slots is None else k_pages.to(self.work)
        work_v = None if slots is None else v_pages.to(self.work)
        PlainOps(self.work).rope_store(holder, None, positions, cos_sin, slots, work_k, work_v, n_q, n_kv, head_dim)
        if slots is not None:
            k_pages.copy_(work_k.to(k_pages.dtype))
            v_pages.copy_(work_v.to(v_pages.dtype))
        return holder[:, :n_q * head_dim].to(weight.dtype).contiguous()

    def fused_norm_gated(self, residual, norm_weight, eps, weight, act=None):
        if norm_weight is None:
            x = residual
        else:
            x = torch.empty(residual.shape, dtype=weight.dtype, device=residual.device)
            self.add_rmsnorm(residual.clone(), None, norm_weight, eps, x)
        gate_up = x.to(self.work) @ weight.to(self.work).t()
        inner = weight.shape[0] // 2
        g, u = gate_up[:, :inner], gate_up[:, inner:]
        if act is not None:
            alpha, limit, shift = (float(v) for v in act)
            g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
            return (g * torch.sigmoid(alpha * g) * (u + shift)).to(weight.dtype)
        return (g * torch.sigmoid(g) * u).to(weight.dtype)

    def linear_add(self, x, weight, bias, residual):
        y = x.to(self.work) @ weight.to(self.work).t()
        if bias is not None:
            y = y + bias.to(self.work)
        residual.add_(y.to(torch.float32))

    def sample(self, logits, temperature, top_p, uniform, out=None, any_cut=True):
        from plain import qwen2_plain as plain
        result = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device) if out is None else out
        for row in range(logits.shape[0]):
            result[row] = plain.sample_token(logits[row].float().cpu().numpy(), float(temperature[row]),
                                             float(top_p[row]), float(uniform[row]))
        return result

    def argmax(self, logits, out=None):
        result = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device) if out is None else out
        for row in range(logits.shape[0]):
            values = logits[row]
            best = values.max()
            hit = torch.nonzero(values == best)
            result[row] = int(hit[0]) if hit.numel() else 0
        return result
