"""Plain PyTorch references of the engine's kernels, one per kernel, with the kernels'
signatures.  They serve two purposes: each GPU kernel is compared with its reference
alone, and on a machine without a GPU the references stand in for the kernel library so
that the engine's bookkeeping (paging, batching, the step function, the scheduler) can be
tested there.  They are test code: the engine itself has no such path.

Everything is computed in float64 and rounded once to the output's type.
"""

from __future__ import annotations

import torch

import plain_lotorax as pl
import plain_ralitar as pr
from plain_model import causal_attention, exponential_race, rms_norm, rope_neox, silu_and_mul, top_k_top_p_filter

WIDE = torch.float64


class PlainKernels:
    name = "plain"

    def embedding(self, table, ids, out):
        out.copy_(table[ids.long()].to(out.dtype))
        return out

    def feed_tokens(self, ids, source, sampled):
        take = source >= 0
        ids[take] = sampled[source[take].long()]
        return ids

    def rmsnorm(self, x, weight, eps, out, residual=None, mode="plain", rows=None):
        xs = x.to(WIDE)
        if rows is not None:
            xs = xs[rows.long()]
        if mode == "add":
            res = residual.to(WIDE)
            summed = xs + (res[rows.long()] if rows is not None else res)
        else:
            summed = xs
        if mode in ("init", "add") and rows is None:
            residual.copy_(summed.to(torch.float32))
            summed = residual.to(WIDE)  # the norm sees what the stream holds
        out.copy_(rms_norm(summed, weight.to(WIDE), eps).to(out.dtype))
        return out

    def silu_mul(self, x, out):
        out.copy_(silu_and_mul(x.to(WIDE)).to(out.dtype))
        return out

    def qk_norm_rope_kv_write(self, qkv, q_out, k_cache, v_cache, q_weight, k_weight, cos, sin, positions, slots,
                              num_heads, num_kv_heads, head_dim, rotary_dim, page_size, eps, write_kv=True):
        t = qkv.shape[0]
        q, k, v = torch.split(qkv.to(WIDE), [num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim], dim=-1)
        q = q.reshape(t, num_heads, head_dim)
        k = k.reshape(t, num_kv_heads, head_dim)
        v = v.reshape(t, num_kv_heads, head_dim)
        if q_weight is not None:
            q = rms_norm(q, q_weight.to(WIDE), eps)
        if k_weight is not None:
            k = rms_norm(k, k_weight.to(WIDE), eps)
        if rotary_dim:
            c = cos[positions.long()].to(WIDE)
            s = sin[positions.long()].to(WIDE)
            q = torch.cat((rope_neox(q[..., :rotary_dim], c, s), q[..., rotary_dim:]), dim=-1)
            k = torch.cat((rope_neox(k[..., :rotary_dim], c, s), k[..., rotary_dim:]), dim=-1)
        q_out.copy_(q.to(q_out.dtype))
        if write_kv:
            for i in range(t):
                slot = int(slots[i])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_cache[page, :, off, :] = k[i].to(k_cache.dtype)
                v_cache[page, :, :, off] = v[i].to(v_cache.dtype)
        return q_out

    def attention_tile_rows(self, dtype, head_dim, page_size, group, max_q_len):
        return 0, 0   # this attention walks tokens, it wants no tiles listed

    def paged_attention(self, q, k_cache, v_cache, out, meta, scale, window=None, parts=None, softcap=None,
                        chunk=None):
        tokens, hq, d = q.shape
        page_size = k_cache.shape[2]
        hkv = k_cache.shape[1]
        for t in range(tokens):
            seq = int(meta.token_seq[t])
            if seq < 0:
                out[t] = 0
                continue
            pos = int(meta.positions[t])
            first = max(0, pos - window + 1) if window else 0
            if chunk:
                first = max(first, pos // chunk * chunk)
            keys = torch.arange(first, pos + 1)
            pages = meta.block_tables[seq].long()[keys // page_size]
            offs = keys % page_size
            k = k_cache[pages, :, offs, :].to(WIDE)        # [n, hkv, d]
            v = v_cache[pages, :, :, offs].to(WIDE)        # [n, hkv, d]
            if softcap:
                for h in range(hq):
                    s = (k[:, h // (hq // hkv)] @ q[t, h].to(WIDE)) * scale
                    s = softcap * torch.tanh(s / softcap)
                    out[t, h] = (torch.softmax(s, dim=0) @ v[:, h // (hq // hkv)]).to(out.dtype)
                continue
            o = causal_attention(q[t:t + 1].to(WIDE), k, v, scale, None, torch.tensor([pos]), keys)
            out[t] = o[0].to(out.dtype)
        return out

    def linear(self, x, weight, bias=None, out_dtype=None, defer=False):
        y = x.to(WIDE) @ weight.to(WIDE).T
        if bias is not None:
            y = y + bias.to(WIDE)
        return y.to(out_dtype or x.dtype)

    def linear_side_by_side(self, xs, weights, out_dtype=None):
        return [self.linear(xs[b], weights[b], None, out_dtype=out_dtype) for b in range(xs.shape[0])]

    def linear_act(self, x, weight, bias, activation, out_dtype=None):
        up = self.linear(x, weight, bias, out_dtype=WIDE)
        return self.unary_act(up, torch.empty(tuple(up.shape), dtype=out_dtype or x.dtype), activation)

    def linear_silu(self, x, weight, bias=None):
        return silu_and_mul(self.linear(x, weight, bias, out_dtype=WIDE)).to(x.dtype)

    def materialize(self, x):
        if hasattr(x, "terms"):    # a sum of scaled terms that a mixer handed on
            out = torch.empty(tuple(x.shape), dtype=torch.float32)
            return self.sum_norm(out, 0.0, x.terms, x.scales, None, 0.0, None)
        return x

    # ---- the kernels of a stream that is normed after every sum, and of attention whose heads are worked together

    def sum_norm(self, stream, alpha, summands, scales, weight, eps, out=None):
        total = alpha * stream.to(WIDE) if alpha != 0 else torch.zeros(tuple(stream.shape), dtype=WIDE)
        for y, s in zip(summands, scales):
            total = total + s * y.to(WIDE)
        if weight is not None:
            total = total / torch.sqrt((total * total).mean(-1, keepdim=True) + eps) * weight.to(WIDE)
        stream.copy_(total.to(stream.dtype))
        if out is not None:
            out.copy_(total.to(out.dtype))
        return stream

    def shift_rows(self, x, mu, out, state, state_off, cu_seqlens_q, slot_of_seq, token_seq):
        width = x.shape[1]
        out.zero_()
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if hi == lo or slot < 0:
                continue
            rows = x[lo:hi].to(WIDE)
            kept = state[slot, state_off:state_off + width]
            before = torch.cat((kept.to(WIDE)[None], rows[:-1]))
            out[lo:hi] = (rows + (before - rows) * mu.to(WIDE)).to(out.dtype)
            kept.copy_(rows[-1].to(kept.dtype))
        return out

    def qkv_rot_write(self, qkv, q_out, k_cache, v_cache, q_weight, k_weight, freq, rot_dims, positions, slots,
                      num_heads, num_kv_heads, head_dim, value_dim, page_size, eps, v_source=None, v_blend=None,
                      v_keep=None):
        t = qkv.shape[0]
        H, G, D, DV = num_heads, num_kv_heads, head_dim, value_dim
        q, k, v = torch.split(qkv.to(WIDE)[:, :(H + G) * D + G * DV], [H * D, G * D, G * DV], dim=-1)
        q, k = q.reshape(t, H, D), k.reshape(t, G, D)
        if q_weight is not None:
            q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.to(WIDE)
        if k_weight is not None:
            k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.to(WIDE)
        if rot_dims:
            half = rot_dims // 2
            a = positions.to(WIDE)[:, None] * freq.to(WIDE)[None]
            c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]

            def turn(x):
                u, w = x[..., :half], x[..., half:rot_dims]
                return torch.cat((u * c - w * s, w * c + u * s, x[..., rot_dims:]), -1)

            q, k = turn(q), turn(k)
        if v_keep is not None:
            v_keep.copy_(v.to(v_keep.dtype))
        if v_source is not None:
            lam = v_blend.to(WIDE)
            v = (1 - lam) * v + lam * v_source.to(WIDE)
        v = v.reshape(t, G, DV)
        q_out.copy_(q.to(q_out.dtype))
        for i in range(t):
            slot = int(slots[i])
            if slot < 0:
                continue
            page, off = divmod(slot, page_size)
            k_cache[page, :, off, :] = k[i].to(k_cache.dtype)
            v_cache[page, :, :, off] = v[i].to(v_cache.dtype)
        return q_out

    def attention_together(self, q, k_cache, v_cache, out, token_seq, positions, block_tables, scale, head_scale=None,
                           sink=None, talk=None, window=None, max_context_len=None, cu_seqlens_q=None, max_q_len=None,
                           parts=None):
        tokens, H, D = q.shape
        G, page_size = k_cache.shape[1], k_cache.shape[2]
        for t in range(tokens):
            seq = int(token_seq[t])
            if seq < 0:
                out[t] = 0
                continue
            pos = int(positions[t])
            first = max(0, pos - window + 1) if window else 0
            keys = torch.arange(first, pos + 1)
            pages = block_tables[seq].long()[keys // page_size]
            offs = keys % page_size
            k = k_cache[pages, :, offs, :].to(WIDE).repeat_interleave(H // G, dim=1)     # [n, H, D]
            v = v_cache[pages, :, :, offs].to(WIDE).repeat_interleave(H // G, dim=1)     # [n, H, DV]
            s = torch.einsum("hd,nhd->hn", q[t].to(WIDE), k) * scale
            if head_scale is not None:
                s = s * head_scale.to(WIDE)[:, None]
            m = s.max(-1, keepdim=True).values
            if sink is not None:
                m = torch.maximum(m, sink.to(WIDE)[:, None])
            e = torch.exp(s - m)
            den = e.sum(-1, keepdim=True)
            if sink is not None:
                den = den + torch.exp(sink.to(WIDE)[:, None] - m)
            w = e / den
            if talk is not None:
                w = talk.to(WIDE) @ w
            out[t] = torch.einsum("hn,nhd->hd", w, v).to(out.dtype)
        return out

    # ---- the kernels of the layer-norm / latent-attention / delta-rule / routed-experts parts

    def layernorm(self, x, weight, bias, eps, out, residual=None, mode="plain", rows=None, next_weight=None,
                  next_bias=None):
        xs = x.to(WIDE)
        w, b = weight.to(WIDE), bias.to(WIDE)
        if rows is not None:
            xs = xs[rows.long()]
        if mode == "post":
            residual.copy_((residual.to(WIDE) + pl.layer_norm(xs, w, b, eps)).to(torch.float32))
            if out is not None:
                out.copy_(pl.layer_norm(residual.to(WIDE), next_weight.to(WIDE), next_bias.to(WIDE), eps).to(out.dtype))
            return out
        if mode == "add":
            res = residual.to(WIDE)
            xs = xs + (res[rows.long()] if rows is not None else res)
        if mode in ("init", "add") and rows is None:
            residual.copy_(xs.to(torch.float32))
            xs = residual.to(WIDE)
        out.copy_(pl.layer_norm(xs, w, b, eps).to(out.dtype))
        return out

    def embedding_scaled(self, table, ids, out, scale):
        out.copy_((table[ids.long()].to(WIDE) * scale).to(out.dtype))
        return out

    def sum_concat(self, hidden, residual, first, out):
        x = hidden.to(WIDE) if residual is None else hidden.to(WIDE) + residual.to(WIDE)
        out.copy_(torch.cat((x, first.to(WIDE)), dim=-1).to(out.dtype))
        return out

    def gated_act(self, x, out, activation):
        g, u = x.to(WIDE).chunk(2, dim=-1)
        f = {"silu": pl.silu, "relu": torch.relu, "gelu_tanh": pl.gelu_tanh}[activation]
        out.copy_((f(g) * u).to(out.dtype))
        return out

    def linear_f32(self, x, weight, bias=None):
        return self.linear(x, weight, bias, out_dtype=torch.float32)

    def latent_prepare(self, proj, q_off, kv_off, heads, dim, rot, rank, rot_dims, norm_weight, eps, freq, mult,
                       positions, slots, pages, q_abs, q_scale):
        T = proj.shape[0]
        p = proj.to(WIDE)
        ang = positions.to(WIDE)[:, None] * freq.to(WIDE)[None, :] if rot_dims else None

        def turn(x):   # x [T, ..., rot]
            if not rot_dims:
                return x
            c, s_ = torch.cos(ang) * mult, torch.sin(ang) * mult
            while c.dim() < x.dim():
                c, s_ = c.unsqueeze(1), s_.unsqueeze(1)
            out = x.clone()
            u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
            out[..., 0:rot_dims:2] = u * c - v * s_
            out[..., 1:rot_dims:2] = v * c + u * s_
            return out

        q = p[:, q_off:q_off + heads * (dim + rot)].reshape(T, heads, dim + rot)
        q_abs[:, :, rank:] = (turn(q[..., dim:]) * q_scale).to(q_abs.dtype)
        if slots is not None:
            c = pl.rms_unit(p[:, kv_off:kv_off + rank], eps) * norm_weight.to(WIDE)
            k = turn(p[:, kv_off + rank:kv_off + rank + rot])
            flat = pages.view(-1, rank + rot)
            for t in range(T):
                if int(slots[t]) >= 0:
                    flat[int(slots[t])] = torch.cat((c[t], k[t])).to(pages.dtype)
        return q_abs

    def heads_gemm(self, x, x_offset, ldx, hsx, weight, y, y_offset, ldy, hsy, heads, m, n, k, alpha=1.0, gate=None,
                   gate_offset=0, ldg=0, exact=False):
        xf, yf = x.reshape(-1), y.view(-1)
        for h in range(heads):
            xs = torch.as_strided(xf, (m, k), (ldx, 1), x_offset + h * hsx).to(WIDE)
            r = alpha * (xs @ weight[h].to(WIDE).T)
            if gate is not None:
                gv = torch.as_strided(gate.reshape(-1), (m,), (ldg,), gate_offset + h).to(WIDE)
                r = r * torch.sigmoid(gv)[:, None]
            torch.as_strided(yf, (m, n), (ldy, 1), y_offset + h * hsy).copy_(r.to(y.dtype))
        return y

    def latent_attention(self, q_abs, pages, out, meta, rank, sink=None, window=None):
        tokens, heads, width = q_abs.shape
        flat = pages.view(-1, width)
        for t in range(tokens):
            seq = int(meta.token_seq[t])
            if seq < 0:
                out[t] = 0
                continue
            pos = int(meta.positions[t])
            first = max(0, pos - window + 1) if window else 0
            keys = torch.arange(first, pos + 1)
            rows = flat[meta.block_tables[seq].long()[keys // meta.page_size] * meta.page_size + keys % meta.page_size].to(WIDE)
            s = q_abs[t].to(WIDE) @ rows.T                                  # [heads, n]
            top = s.max(dim=-1, keepdim=True).values
            if sink is not None:
                top = torch.maximum(top, sink.to(WIDE)[:, None])
            e = torch.exp(s - top)
            denom = e.sum(dim=-1, keepdim=True)
            if sink is not None:
                denom = denom + torch.exp(sink.to(WIDE)[:, None] - top)
            out[t] = ((e / denom) @ rows[:, :rank]).to(out.dtype)
        return out

    def conv_silu_state(self, x, channels, taps_weight, state, cu_seqlens_q, slot_of_seq, out, max_q_len=None,
                        bias=None, activation="silu", x_offset=0):
        taps = taps_weight.shape[1]
        x = x[:, x_offset:]
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if slot < 0:
                out[lo:hi] = 0
                continue
            tail = state[slot, :(taps - 1) * channels].view(taps - 1, channels)
            y, new_tail = pl.short_convolution(x[lo:hi, :channels].to(WIDE), taps_weight.to(WIDE), tail.to(WIDE))
            if bias is not None:
                y = y + bias.to(WIDE)
            out[lo:hi] = (pl.silu(y) if activation == "silu" else y).to(out.dtype)
            tail.copy_(new_tail.to(tail.dtype))
        return out

    def delta_rule(self, qkv, gates, a_off, b_off, a_log, dt_bias, state, state_off, cu_seqlens_q, slot_of_seq, out,
                   heads, kv_heads, dim, vdim, decay=None, per_channel=False):
        if per_channel:
            return self._delta_rule_channels(qkv, gates, a_off, b_off, a_log, dt_bias, state, state_off, cu_seqlens_q,
                                             slot_of_seq, out, heads, kv_heads, dim, vdim,
                                             gates if decay is None else decay)
        if decay is not None:
            gates = torch.cat((gates, decay), dim=1)
            a_off = gates.shape[1] - decay.shape[1] + a_off
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if slot < 0:
                out[lo:hi] = 0
                continue
            n = hi - lo
            x = qkv[lo:hi].to(WIDE)
            q = x[:, :kv_heads * dim].reshape(n, kv_heads, dim)
            k = x[:, kv_heads * dim:2 * kv_heads * dim].reshape(n, kv_heads, dim)
            v = x[:, 2 * kv_heads * dim:].reshape(n, heads, vdim)
            q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
            k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            gs = gates[lo:hi].to(WIDE)
            beta = torch.sigmoid(gs[:, b_off:b_off + heads])
            g = torch.exp(-torch.exp(a_log.to(WIDE)) * pl.softplus(gs[:, a_off:a_off + heads] + dt_bias.to(WIDE)))
            S = state[slot, state_off:state_off + heads * dim * vdim].view(heads, dim, vdim)
            for h in range(heads):
                kv = h // (heads // kv_heads)
                o, new = pl.delta_rule(q[:, kv], k[:, kv], v[:, h], beta[:, h], g[:, h], S[h].to(WIDE))
                out[lo:hi, h] = o.to(out.dtype)
                S[h] = new.to(S.dtype)
        return out

    def _delta_rule_channels(self, qkv, gates, a_off, b_off, a_log, dt_bias, state, state_off, cu_seqlens_q,
                             slot_of_seq, out, heads, kv_heads, dim, vdim, decay):
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if slot < 0:
                out[lo:hi] = 0
                continue
            n = hi - lo
            x = qkv[lo:hi].to(WIDE)
            q = x[:, :kv_heads * dim].reshape(n, kv_heads, dim)
            k = x[:, kv_heads * dim:2 * kv_heads * dim].reshape(n, kv_heads, dim)
            v = x[:, 2 * kv_heads * dim:].reshape(n, heads, vdim)
            q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
            k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            beta = torch.sigmoid(gates[lo:hi, b_off:b_off + heads].to(WIDE))
            raw = decay[lo:hi, a_off:a_off + heads * dim].to(WIDE) + dt_bias.to(WIDE)
            g = torch.exp(-torch.exp(a_log.to(WIDE)).view(1, heads, 1) * pr.softplus(raw).view(n, heads, dim))
            S = state[slot, state_off:state_off + heads * dim * vdim].view(heads, dim, vdim)
            for h in range(heads):
                kv = h // (heads // kv_heads)
                cur = S[h].to(WIDE)
                for t in range(n):
                    o, cur = pr.delta_step(cur, q[t, kv], k[t, kv], v[t, h], beta[t, h], g[t, h])
                    out[lo + t, h] = o.to(out.dtype)
                S[h] = cur.to(S.dtype)
        return out

    def delta_out(self, o, gates, gate_off, weight, eps, out, activation="silu"):
        tokens, heads, vdim = o.shape
        g = gates[:, gate_off:gate_off + heads * vdim].to(WIDE).view(tokens, heads, vdim)
        y = pl.rms_unit(o.to(WIDE), eps) * weight.to(WIDE) * (pl.silu(g) if activation == "silu" else torch.sigmoid(g))
        out.copy_(y.reshape(tokens, heads * vdim).to(out.dtype))
        return out

    # ---- the kernels of the float32-stream block, the pair embedding, the gated recurrence and key-value attention

    def embedding_bigram(self, table, pairs, ids, state, cu_seqlens_q, slot_of_seq, token_seq, out, buckets, mul_prev,
                         mul_cur):
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if hi <= lo:
                continue
            if slot < 0:
                out[lo:hi] = 0
                continue
            prev = int(state[slot, 0]) - 1
            for t in range(lo, hi):
                cur = int(ids[t])
                row = buckets if prev < 0 else (prev * mul_prev + cur * mul_cur) % buckets
                out[t] = (table[cur].to(WIDE) + pairs[row].to(WIDE)).to(out.dtype)
                prev = cur
            state[slot, 0] = prev + 1
        return out

    def rmsnorm_post(self, x, weight, eps, stream, out=None):
        stream.copy_((stream.to(WIDE) + pr.rms(x.to(WIDE), eps) * weight.to(WIDE)).to(stream.dtype))
        if out is not None:
            out.copy_(stream.to(out.dtype))
        return out

    def rmsnorm_rows(self, x, weight, eps, rows, out):
        src = x if rows is None else x[rows.long()]
        out.copy_((pr.rms(src.to(WIDE), eps) * weight.to(WIDE)).to(out.dtype))
        return out

    def stream_norm(self, stream, x, weight, eps, out, init=False):
        stream.copy_(x.to(torch.float32) if init else (stream.to(WIDE) + x.to(WIDE)).to(torch.float32))
        out.copy_((pr.rms(stream.to(WIDE), eps) * weight.to(WIDE)).to(out.dtype))
        return out

    # ---- linear recurrences with a matrix state, attention without rotation, and what stands around them

    def linear_scan(self, r, r_off, r_heads, k, k_off, k_heads, v, v_off, w, w_off, state, state_off, cu_seqlens_q,
                    slot_of_seq, out, heads, dim, vdim, per_channel=True, w_bias=None, v_scale=None, bonus=None,
                    skip=None, max_q_len=None, step_bias=None, a_log=None):
        if a_log is not None:      # raw step sizes in w's place: the steps multiply v, the decays follow from them
            steps = pl.softplus(w[:, w_off:w_off + heads].to(WIDE) + step_bias.to(WIDE))
            w, w_off, v_scale = torch.exp(-torch.exp(a_log.to(WIDE)) * steps), 0, steps
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if slot < 0:
                out[lo:hi] = 0
                continue
            n = hi - lo
            rr = r[lo:hi, r_off:r_off + r_heads * dim].to(WIDE).reshape(n, r_heads, dim)
            kk = k[lo:hi, k_off:k_off + k_heads * dim].to(WIDE).reshape(n, k_heads, dim)
            vv = v[lo:hi, v_off:v_off + heads * vdim].to(WIDE).reshape(n, heads, vdim)
            if per_channel:
                ww = w[lo:hi, w_off:w_off + heads * dim].to(WIDE)
                if w_bias is not None:
                    ww = torch.exp(-torch.exp(ww + w_bias.to(WIDE)))
                ww = ww.reshape(n, heads, dim)
            else:
                ww = w[lo:hi, w_off:w_off + heads].to(WIDE)[:, :, None].expand(n, heads, dim)
            S = state[slot, state_off:state_off + heads * dim * vdim].view(heads, dim, vdim)
            cur = S.to(WIDE)
            res = torch.zeros(n, heads, vdim, dtype=WIDE)
            for t in range(n):
                for h in range(heads):
                    rh, kh = rr[t, h // (heads // r_heads)], kk[t, h // (heads // k_heads)]
                    vin = vv[t, h] * (v_scale[lo + t, h].to(WIDE) if v_scale is not None else 1.0)
                    kv = torch.outer(kh, vin)
                    if bonus is not None:
                        res[t, h] = (cur[h] + bonus[h].to(WIDE)[:, None] * kv).T @ rh
                        cur[h] = ww[t, h][:, None] * cur[h] + kv
                    else:
                        cur[h] = ww[t, h][:, None] * cur[h] + kv
                        res[t, h] = cur[h].T @ rh
                    if skip is not None:
                        res[t, h] += skip[h].to(WIDE) * vv[t, h]
            S.copy_(cur.to(S.dtype))
            out[lo:hi] = res.reshape(n, heads * vdim).to(out.dtype)
        return out

    def token_shift(self, x, mu, mixes, state, state_off, cu_seqlens_q, slot_of_seq, token_seq):
        width = x.shape[1]
        mixes.zero_()
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if hi == lo:
                continue
            rows = x[lo:hi].to(WIDE)
            kept = state[slot, state_off:state_off + width] if slot >= 0 else torch.zeros(width)
            before = torch.cat((kept.to(WIDE)[None], rows[:-1]))
            for s in range(mu.shape[0]):
                mixes[s, lo:hi] = (rows + (before - rows) * mu[s].to(WIDE)).to(mixes.dtype)
            if slot >= 0:
                kept.copy_(rows[-1].to(kept.dtype))
        return mixes

    def step_decay(self, raw, raw_off, dt_bias, a_log, dt, decay):
        heads = dt.shape[1]
        step = pl.softplus(raw[:, raw_off:raw_off + heads].to(WIDE) + dt_bias.to(WIDE))
        dt.copy_(step.to(dt.dtype))
        decay.copy_(torch.exp(-torch.exp(a_log.to(WIDE)) * step).to(decay.dtype))
        return dt, decay

    def group_norm_gate(self, y, groups, weight, eps, out, gate=None, gate_off=0, gate_first=False):
        tokens, width = y.shape
        z = y.to(WIDE)
        g = pl.silu(gate[:, gate_off:gate_off + width].to(WIDE)) if gate is not None else None
        if g is not None and gate_first:
            z = z * g
        z = pr.rms(z.reshape(tokens, groups, width // groups), eps).reshape(tokens, width)
        if weight is not None:
            z = z * weight.to(WIDE)
        if g is not None and not gate_first:
            z = z * g
        out.copy_(z.to(out.dtype))
        return out

    def qkv_plain_write(self, proj, q_out, k_cache, v_cache, positions, slots, num_heads, num_kv_heads, head_dim,
                        value_dim, page_size, unit_norm, eps, temperature=None, write_kv=True):
        t = proj.shape[0]
        q, k, v = torch.split(proj.to(WIDE), [num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * value_dim],
                              dim=-1)
        q = q.reshape(t, num_heads, head_dim)
        k = k.reshape(t, num_kv_heads, head_dim)
        v = v.reshape(t, num_kv_heads, value_dim)
        if unit_norm:
            q, k = pr.rms(q, eps), pr.rms(k, eps)
        if temperature is not None and temperature[0] != 0:
            steps = torch.div(positions.long() + 1, int(temperature[1]), rounding_mode="floor").to(WIDE)
            q = q * (1 + temperature[0] * torch.log(steps + 1))[:, None, None]
        q_out.zero_()
        q_out[:, :, :head_dim] = q.to(q_out.dtype)
        if write_kv:
            for i in range(t):
                slot = int(slots[i])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_cache[page, :, off, :head_dim] = k[i].to(k_cache.dtype)
                v_cache[page, :, :value_dim, off] = v[i].to(v_cache.dtype)
        return q_out

    def narrow_heads(self, x, value_dim):
        return x[:, :, :value_dim].reshape(x.shape[0], -1).contiguous()

    def mean_of_norms(self, xs, weights, eps, out):
        total = sum(pr.rms(x.to(WIDE), eps) * w.to(WIDE) for x, w in zip(xs, weights))
        out.copy_((total / len(xs)).to(out.dtype))
        return out

    def embedding_positions(self, table, rows, ids, positions, out):
        out.copy_((table[ids.long()].to(WIDE) + rows[positions.long()].to(WIDE)).to(out.dtype))
        return out

    def unary_act(self, x, out, activation):
        z = x.to(WIDE)
        y = {"silu": pl.silu, "relu": torch.relu, "gelu_tanh": pl.gelu_tanh, "tanh": torch.tanh,
             "relu_squared": lambda a: torch.relu(a) ** 2}[activation](z)
        out.copy_(y.to(out.dtype))
        return out

    def stream_add(self, stream, x, init=False):
        stream.copy_(x.to(torch.float32) if init else (stream.to(WIDE) + x.to(WIDE)).to(torch.float32))
        return stream

    def scale_rows(self, x, scale):
        x.mul_(scale)
        return x

    def cast_rows(self, x, dtype):
        return x.to(dtype)

    def token_gate(self, raw, table, col_off, ids, out):
        e = table[ids.long(), col_off:col_off + raw.shape[1]].to(WIDE)
        out.copy_((pr.gelu_tanh(raw.to(WIDE)) * e).to(out.dtype))
        return out

    def rglru_scan(self, u, gates, ra_bias, ri_bias, lam, proj, y_off, state, state_off, cu_seqlens_q, slot_of_seq, out,
                   decay_scale, max_q_len=None):
        c = u.shape[1]
        sp = pr.softplus(lam.to(WIDE))
        for b in range(slot_of_seq.numel()):
            lo, hi, slot = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1]), int(slot_of_seq[b])
            if slot < 0:
                out[lo:hi] = 0
                continue
            S = state[slot, state_off:state_off + c].to(WIDE)
            for t in range(lo, hi):
                r = torch.sigmoid(gates[0, t].to(WIDE) + ra_bias.to(WIDE).reshape(-1))
                i = torch.sigmoid(gates[1, t].to(WIDE) + ri_bias.to(WIDE).reshape(-1))
                a = torch.exp(-decay_scale * r * sp)
                S = a * S + torch.sqrt(1 - a * a) * (i * u[t].to(WIDE))
                out[t] = (S * pr.gelu_tanh(proj[t, y_off:y_off + c].to(WIDE))).to(out.dtype)
            state[slot, state_off:state_off + c] = S.to(state.dtype)
        return out

    def keys_as_values_write(self, proj, q_out, k_cache, v_cache, q_weight, k_weight, freq, rot_dims, positions, slots,
                             num_heads, num_kv_heads, head_dim, page_size, eps, write_kv=True):
        t = proj.shape[0]
        qn, kn = num_heads * head_dim, num_kv_heads * head_dim
        q, k = proj[:, :qn].to(WIDE), proj[:, qn:qn + kn].to(WIDE)
        v = k.reshape(t, num_kv_heads, head_dim)
        if q_weight is not None:
            q = pr.rms(q, eps) * q_weight.to(WIDE)
        if k_weight is not None:
            k = pr.rms(k, eps) * k_weight.to(WIDE)
        q, k = q.reshape(t, num_heads, head_dim), k.reshape(t, num_kv_heads, head_dim)
        if rot_dims:
            q, k = pr.rotate_pairs(q, positions, freq.to(WIDE)), pr.rotate_pairs(k, positions, freq.to(WIDE))
        q_out.copy_(q.to(q_out.dtype))
        if write_kv:
            for i in range(t):
                slot = int(slots[i])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_cache[page, :, off, :] = k[i].to(k_cache.dtype)
                v_cache[page, :, :, off] = v[i].to(v_cache.dtype)
        return q_out

    def sigmoid_gate(self, x, gates, gate_off, out):
        g = gates[:, gate_off:gate_off + x.shape[1]].to(WIDE)
        out.copy_((x.to(WIDE) * torch.sigmoid(g)).to(out.dtype))
        return out

    def router_choose(self, logits, correction, top, renormalize=False):
        s = torch.sigmoid(logits.to(WIDE))
        pick = s + correction.to(WIDE) if correction is not None else s
        ids = torch.topk(pick, top, dim=-1).indices
        w = torch.gather(s, 1, ids)
        if renormalize:
            w = w / w.sum(dim=-1, keepdim=True)
        return ids.to(torch.int32), w.to(torch.float32)

    def experts_forward(self, x, gate_up, down, ids, weights, activation="silu"):
        f = {"silu": pl.silu, "relu": torch.relu, "gelu_tanh": pl.gelu_tanh}[activation]
        xs = x.to(WIDE)
        y = torch.zeros(xs.shape, dtype=WIDE)
        ff = gate_up.shape[1] // 2
        for t in range(xs.shape[0]):
            for k in range(ids.shape[1]):
                e = int(ids[t, k])
                both = gate_up[e].to(WIDE) @ xs[t]
                y[t] += float(weights[t, k]) * (down[e].to(WIDE) @ (f(both[:ff]) * both[ff:]))
        return y.to(x.dtype)

    def exponential_noise(self, seeds, counters, vocab):
        rows = []
        for s, c in zip(seeds.tolist(), counters.tolist()):
            rows.append(exponential_noise_row(s, c, vocab))
        return torch.stack(rows)

    def sample(self, logits, temperatures, out, top_ks=None, top_ps=None, noise=None, seeds=None, counters=None,
               eps=1e-10):
        rows, vocab = logits.shape
        for r in range(rows):
            temp = float(temperatures[r]) if temperatures is not None else 0.0
            if not temp > 0:
                out[r] = int(logits[r].argmax())
                continue
            if noise is not None:
                e = noise[r if noise.shape[0] == rows and rows > 1 else 0]
            else:
                e = exponential_noise_row(int(seeds[r]), int(counters[r]), vocab)
            k = int(top_ks[r]) if top_ks is not None else -1
            p = float(top_ps[r]) if top_ps is not None else 1.0
            if (k > 0 and k < vocab) or p < 1.0:
                probs = torch.softmax(logits[r].to(WIDE) / temp, dim=-1)
                kept = top_k_top_p_filter(probs, k if 0 < k < vocab else -1, p)
                out[r] = int((kept / (e.to(WIDE) + eps)).argmax())
            else:
                out[r] = int(exponential_race(logits[r:r + 1], torch.tensor([temp]), e.unsqueeze(0), eps)[0])
        return out


_M64 = (1 << 64) - 1


def _mix64(x: int) -> int:
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _M64
    return x ^ (x >> 31)


def exponential_noise_row(seed: int, counter: int, vocab: int) -> torch.Tensor:
    """The engine's noise: Exp(1) draws from an integer mix of (seed, counter, token)."""
    import math

    base = _mix64((seed ^ ((counter * 0x9E3779B97F4A7C15) & _M64)) & _M64)
    out = []
    for v in range(vocab):
        z = _mix64((base + (v + 1) * 0xD6E8FEB86659FD93) & _M64)
        u = (float(z >> 40) + 0.5) / 16777216.0
        out.append(-math.log(u))
    return torch.tensor(out, dtype=torch.float32)
