"""Plain PyTorch versions of the kernel operations, one per kernel, with the same
signatures as ``tempura_amd.kernels.ops``.  They serve two purposes in tests only:
(1) the reference each HIP kernel is graded against on its own; (2) a host stand-in
installed with ``ops.set_backend`` so that the engine's bookkeeping (pages, batching,
cutting) can be tested without a GPU.  Everything is computed in float64 and rounded
to the requested dtype at the end.
"""
from __future__ import annotations

import torch


class EmuOps:
    def embed(self, tokens, table, positions=None, inv_freq=None, streams=1):
        x = table[tokens.long()].double()
        if inv_freq is not None:
            ang = positions.double()[:, None] * inv_freq.double()[None, :]
            pe = torch.stack([torch.sin(ang), torch.cos(ang)], dim=2).reshape(x.shape[0], -1)[:, : x.shape[1]]
            x = x + pe
        return x.to(torch.float32).repeat(1, streams)

    def stream_step(self, h, streams, y=None, mix=None, out_coef=None, in_coef=None, norm_weight=None, eps=0.0,
                    out_dtype=None, rows=None, write_back=True):
        n, width = h.shape[0], h.shape[1] // streams
        hs = h.double().reshape(n, streams, width)
        if y is not None:
            m = torch.eye(streams, dtype=torch.float64) if mix is None else mix.double().reshape(streams, streams)
            o = torch.ones(streams, dtype=torch.float64) if out_coef is None else out_coef.double()
            hs = torch.einsum("ab,naw->nbw", m, hs) + o[None, :, None] * y.double()[:, None, :]
            if write_back:
                h.copy_(hs.reshape(n, -1).to(torch.float32))
                hs = h.double().reshape(n, streams, width)
        if out_dtype is None:
            return None
        c = torch.ones(streams, dtype=torch.float64) if in_coef is None else in_coef.double()
        u = torch.einsum("a,naw->nw", c, hs)
        if rows is not None:
            u = u[rows.long()]
        if norm_weight is not None:
            u = u / torch.sqrt((u * u).mean(dim=-1, keepdim=True) + eps) * norm_weight.double()
        return u.to(out_dtype)

    def scale_(self, x, scale):
        x.mul_(scale)
        return x

    def gated_act(self, gu, out_dtype, slope=1.0, limit=0.0, up_offset=0.0, interleaved=False):
        i = gu.shape[1] // 2
        if interleaved:
            y = gu.double().reshape(gu.shape[0], -1, 2, 8)
            g, u = y[:, :, 0].reshape(gu.shape[0], -1), y[:, :, 1].reshape(gu.shape[0], -1)
        else:
            g, u = gu.double()[:, :i], gu.double()[:, i:]
        if limit > 0:
            g = torch.clamp(g, max=limit)
            u = torch.clamp(u, -limit, limit)
        return (g * torch.sigmoid(slope * g) * (u + up_offset)).to(out_dtype)

    def qk_store(self, rows, q_bias, k_bias, slots, num_heads, num_kv_heads, head_dim, k_cache, v_cache, q_dtype):
        n = rows.shape[0]
        q_dim = num_heads * head_dim
        q = rows.double()[:, :q_dim]
        if q_bias is not None:
            q = q + q_bias.double()
        if slots is not None:
            k = rows.double()[:, q_dim:]
            if k_bias is not None:
                k = k + k_bias.double()
            k = k.reshape(n, num_kv_heads, head_dim)
            ps = k_cache.shape[2]
            page, off = slots.long() // ps, slots.long() % ps
            k_cache[page, :, off] = k.to(k_cache.dtype)
            if v_cache is not None:
                v_cache[page, :, :, off] = k.to(v_cache.dtype)
        return q.reshape(n, num_heads, head_dim).to(q_dtype).contiguous()

    def causal_conv(self, proj, col0, channels, weight, bias, state, cu_seqlens, token_req, state_slots, num_requests,
                    state_off=0, act=True):
        taps = weight.shape[0]                    # tap-major: [taps, channels]
        out = torch.zeros(proj.shape[0], channels, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        b = torch.zeros(channels, dtype=torch.float64) if bias is None else bias.double()
        lo, hi = state_off, state_off + (taps - 1) * channels
        for r in range(num_requests):
            a, e = cu[r], cu[r + 1]
            if e <= a:
                continue
            slot = int(state_slots[r])
            carried = state[slot, lo:hi].double().reshape(taps - 1, channels)
            seq = torch.cat([carried, proj[a:e, col0: col0 + channels].double()], dim=0)
            for t in range(e - a):
                out[a + t] = (seq[t: t + taps] * weight.double()).sum(0) + b
            state[slot, lo:hi] = seq[seq.shape[0] - (taps - 1):].reshape(-1).to(torch.float32)
        return (out * torch.sigmoid(out) if act else out).to(torch.float32)

    def ssm_scan(self, xbc, proj, dt_col0, dt_bias, a_log, d_skip, state, state_off, cu_seqlens, state_slots, num_requests,
                 num_heads, head_dim, state_size, groups, max_run=None):
        n = xbc.shape[0]
        H, P, N, G = num_heads, head_dim, state_size, groups
        inner = H * P
        x = xbc.double()[:, :inner].reshape(n, H, P)
        Bm = xbc.double()[:, inner: inner + G * N].reshape(n, G, N).repeat_interleave(H // G, dim=1)
        Cm = xbc.double()[:, inner + G * N:].reshape(n, G, N).repeat_interleave(H // G, dim=1)
        dt = torch.nn.functional.softplus(proj.double()[:, dt_col0: dt_col0 + H] + dt_bias.double())
        decay = torch.exp(-torch.exp(a_log.double()) * dt)
        y = torch.zeros(n, H, P, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        for r in range(num_requests):
            slot = int(state_slots[r])
            S = state[slot, state_off: state_off + H * N * P].double().reshape(H, N, P)
            for t in range(cu[r], cu[r + 1]):
                S = decay[t, :, None, None] * S + dt[t, :, None, None] * Bm[t, :, :, None] * x[t, :, None, :]
                y[t] = torch.einsum("hnp,hn->hp", S, Cm[t]) + d_skip.double()[:, None] * x[t]
            state[slot, state_off: state_off + H * N * P] = S.reshape(-1).to(torch.float32)
        return y.reshape(n, inner).to(torch.float32)

    def gated_group_norm(self, y, proj, z_col0, weight, eps, groups, out_dtype):
        n, inner = y.shape
        z = proj.double()[:, z_col0: z_col0 + inner]
        v = (y.double() * z * torch.sigmoid(z)).reshape(n, groups, inner // groups)
        v = v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
        return (v.reshape(n, inner) * weight.double()).to(out_dtype)

    def rmsnorm(self, h, weight, eps, out_dtype, rows=None, groups=1):
        x = h.double()
        if rows is not None:
            x = x[rows.long()]
        p = x.reshape(x.shape[0], groups, x.shape[1] // groups)
        y = (p * (1.0 / torch.sqrt((p * p).mean(dim=-1, keepdim=True) + eps))).reshape(x.shape) * weight.double()
        return y.to(out_dtype)

    def rmsnorm_cols(self, x, col0, width, weight, eps, out_dtype, groups=1):
        return self.rmsnorm(x[:, col0: col0 + width], weight, eps, out_dtype, None, groups)

    def residual_conv(self, x, weight, state, state_off, cu_seqlens, token_req, state_slots, num_requests, out_dtype):
        subs, taps, width = weight.shape
        out = torch.zeros(subs, x.shape[0], width, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        lo, hi = state_off, state_off + (taps - 1) * width
        for r in range(num_requests):
            a, e = cu[r], cu[r + 1]
            if e <= a:
                continue
            slot = int(state_slots[r])
            carried = state[slot, lo:hi].double().reshape(taps - 1, width) if taps > 1 else torch.zeros(0, width, dtype=torch.float64)
            seq = torch.cat([carried, x[a:e].double()], dim=0)
            for t in range(e - a):
                for sub in range(subs):
                    out[sub, a + t] = seq[t + taps - 1] + (seq[t: t + taps] * weight[sub].double()).sum(0)
            if taps > 1:
                state[slot, lo:hi] = seq[seq.shape[0] - (taps - 1):].reshape(-1).to(torch.float32)
        return [out[sub].to(out_dtype) for sub in range(subs)]

    def add_row(self, h, table, row):
        h.add_(table[row])

    def general_delta_scan(self, proj, col0, decay, a_bias, state, state_off, cu_seqlens, state_slots, num_requests, heads, dim, unit_eps):
        n, hd = proj.shape[0], heads * dim
        x = proj.double()
        r, k, v, ar = (x[:, col0 + i * hd: col0 + (i + 1) * hd].reshape(n, heads, dim) for i in range(4))
        a = torch.sigmoid(ar + a_bias.double().reshape(heads, dim))
        w = decay.double().reshape(n, heads, dim)
        y = torch.zeros(n, heads, dim, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        for q in range(num_requests):
            slot = int(state_slots[q])
            # (kept column by column: [heads, value, key])
            S = state[slot, state_off: state_off + hd * dim].double().reshape(heads, dim, dim).transpose(1, 2).clone()
            for t in range(cu[q], cu[q + 1]):
                u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + unit_eps)
                seen = torch.einsum("hd,hdv->hv", u, S)
                S = w[t][:, :, None] * S - (a[t] * u)[:, :, None] * seen[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
                y[t] = torch.einsum("hdv,hd->hv", S, r[t])
            state[slot, state_off: state_off + hd * dim] = S.transpose(1, 2).reshape(-1).to(torch.float32)
        return y.reshape(n, hd).to(torch.float32)

    def latent_rows(self, proj, q_col0, rot_col0, up, heads, dim, rot, vdim):
        n, key = proj.shape[0], rot + dim
        q = proj[:, q_col0: q_col0 + heads * key]
        shared = proj[:, rot_col0: rot_col0 + rot][:, None, :].expand(n, heads, rot)
        k = torch.cat([shared, up[:, : heads * dim].reshape(n, heads, dim)], dim=2).reshape(n, heads * key)
        return torch.cat([q, k, up[:, heads * dim: heads * (dim + vdim)]], dim=1).to(torch.float32).contiguous()

    def split_norm_ok(self, m, width, dtype):
        return dtype == torch.bfloat16 and 0 < m <= 128 and width % 32 == 0

    @staticmethod
    def _rows(x):
        """Plain rows, or handed-over rows (x = bfloat16(h * weight), ss = sums of squares per 16 columns)
        with the factor that finishes their norm."""
        from tempura_amd.kernels.ops import KBlocked, Prenormed
        if isinstance(x, KBlocked):
            return x.row_major().double(), 1.0
        if isinstance(x, Prenormed):
            rstd = torch.rsqrt(x.ss.double().sum(0)[: x.x.shape[0]] / x.x.shape[1] + x.eps)
            return x.x.double(), rstd[:, None]
        return x.double(), 1.0

    def linear(self, x, w, out_dtype, residual=None, next_norm=None):
        from tempura_amd.kernels.ops import Prenormed
        xd, scale = self._rows(x)
        y = (xd @ w.double().T) * scale
        if residual is not None:
            residual.copy_((residual.double() + y).to(torch.float32))
            if next_norm is None:
                return residual
            m, n = residual.shape
            if not (self.split_norm_ok(m, n, x.dtype if torch.is_tensor(x) else torch.bfloat16) and xd.shape[1] % 32 == 0):
                return residual, None
            weight, eps = next_norm
            if m > 16:       # the kernel that adds the product into the residual norms the rows as well
                return residual, self.rmsnorm(residual, weight, eps, torch.bfloat16)
            ss = torch.zeros(((n + 15) // 16, 16), dtype=torch.float32)
            sq = torch.nn.functional.pad(residual.double() ** 2, (0, ss.shape[0] * 16 - n))
            ss[:, :m] = sq.reshape(m, -1, 16).sum(2).T.to(torch.float32)
            return residual, Prenormed((residual * weight).to(torch.bfloat16), ss, eps)
        return y.to(out_dtype)

    def linear_swiglu(self, x, w, blocked_out=False, slope=1.0, limit=0.0, up_offset=0.0):
        from tempura_amd.kernels.ops import KBlocked
        xd, scale = self._rows(x)
        x = xd
        y = ((x @ w.double().T) * scale).reshape(x.shape[0], -1, 2, 8)      # eight gate rows, eight up rows in turn
        g, u = y[:, :, 0].reshape(x.shape[0], -1), y[:, :, 1].reshape(x.shape[0], -1)
        if limit > 0:
            g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
        out = (g / (1.0 + torch.exp(-slope * g)) * (u + up_offset)).to(torch.bfloat16)
        m, i = out.shape
        if blocked_out and 0 < m <= 16 and i % 32 == 0:
            return KBlocked(out.reshape(m, i // 8, 8).permute(1, 0, 2).contiguous(), m, i)
        return out

    def rope_kv_write(self, qkv, positions, slots, inv_freq, rotary_dim, factor, num_heads, num_kv_heads,
                      head_dim, k_cache, v_cache, q_dtype, value_dim=None, pad_dim=None):
        n = qkv.shape[0]
        nrot = num_heads + (num_kv_heads if slots is not None else 0)
        x = qkv.double()[:, : nrot * head_dim].reshape(n, nrot, head_dim).clone()
        if rotary_dim:
            half = rotary_dim // 2
            ang = positions.double()[:, None] * inv_freq.double()[None, :]
            c = (torch.cos(ang) * factor)[:, None, :]
            s = (torch.sin(ang) * factor)[:, None, :]
            # paired order: elements (2 d, 2 d + 1) rotate together by the angle of pair d
            x0, x1 = x[..., 0:rotary_dim:2].clone(), x[..., 1:rotary_dim:2].clone()
            x[..., 0:rotary_dim:2] = x0 * c - x1 * s
            x[..., 1:rotary_dim:2] = x0 * s + x1 * c
        if pad_dim is not None and pad_dim > head_dim:      # zeros behind every head's own elements
            x = torch.nn.functional.pad(x, (0, pad_dim - head_dim))
        q = x[:, :num_heads].to(q_dtype).contiguous()
        if slots is not None:
            k = x[:, num_heads:]
            v = qkv.double()[:, nrot * head_dim:].reshape(n, num_kv_heads, value_dim or head_dim)
            ps = k_cache.shape[2]
            page, off = slots.long() // ps, slots.long() % ps
            k_cache[page, :, off] = k.to(k_cache.dtype)
            v_cache[page, :, :, off] = v.to(v_cache.dtype)          # values are kept transposed
        return q

    def paged_attention(self, q, k_cache, v_cache, block_tables, cu_seqlens, context_lens, token_req, scale,
                        window, max_q_len, max_context_len, num_single=None, dist_bias=None, sink=None, keep_first=0):
        n, heads, d = q.shape
        kvh, ps = k_cache.shape[1], k_cache.shape[2]
        group = heads // kvh
        vd = v_cache.shape[2]
        out = torch.zeros(n, heads, vd, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        for r in range(block_tables.shape[0]):
            qs, qe = cu[r], cu[r + 1]
            ctx = int(context_lens[r])
            pages = block_tables[r].long()
            j = torch.arange(ctx)
            rows_page, rows_off = pages[j // ps], j % ps
            K = k_cache[rows_page, :, rows_off].double()      # [ctx, kvh, d]
            V = v_cache[rows_page, :, :, rows_off].double()      # [ctx, kvh, d]
            for t in range(qs, qe):
                pos = ctx - (qe - qs) + (t - qs)
                lo = max(0, pos - window + 1) if window > 0 else 0
                # (the keys a query sees: the window, and under a window the request's first keep_first keys)
                seen = torch.cat([torch.arange(0, min(keep_first, lo) if window > 0 else 0), torch.arange(lo, pos + 1)])
                for h in range(heads):
                    sc = (K[seen, h // group] @ q[t, h].double()) * scale
                    if dist_bias is not None:
                        dist = torch.clamp(pos - seen, max=dist_bias.shape[1] - 1)
                        sc = sc + dist_bias[h].double()[dist]
                    if sink is not None:
                        p = torch.softmax(torch.cat([sc, sink[h].double().reshape(1)]), dim=0)[:-1]
                    else:
                        p = torch.softmax(sc, dim=0)
                    out[t, h] = p @ V[seen, h // group]
        return out.reshape(n, heads * vd).to(q.dtype)

    def embed_bigram(self, tokens, table, bigram, positions, token_req, cu_seqlens, state_slots, prev_state, num_requests,
                     mul_prev, mul_cur, buckets, scale=1.0, pos_table=None):
        out = torch.zeros(tokens.numel(), table.shape[1], dtype=torch.float64)
        cu = cu_seqlens.tolist()
        for r in range(num_requests):
            slot = int(state_slots[r])
            for t in range(cu[r], cu[r + 1]):
                tok = int(tokens[t])
                out[t] = table[tok].double() * scale
                if bigram is not None:
                    if int(positions[t]) == 0:
                        row = buckets
                    else:
                        prev = int(tokens[t - 1]) if t > cu[r] else int(prev_state[slot].reshape(-1)[0])
                        row = (prev * mul_prev + tok * mul_cur) % buckets
                    out[t] += bigram[row].double()
                if pos_table is not None:
                    out[t] += pos_table[int(positions[t])].double()
            if cu[r + 1] > cu[r] and bigram is not None:
                prev_state[slot] = int(tokens[cu[r + 1] - 1])
        return out.to(torch.float32)

    def sigmoid_gate(self, a, proj, gate_col0, scale, out, out_col0):
        v = a.double()
        if proj is not None:
            v = v * torch.sigmoid(proj.double()[:, gate_col0: gate_col0 + a.shape[1]])
        out[:, out_col0: out_col0 + a.shape[1]] = (v * scale).to(out.dtype)

    def norm_add(self, h, y, weight, eps, next_weight=None, next_eps=0.0, out_dtype=None):
        yd = y.double()
        h.copy_((h.double() + yd / torch.sqrt((yd * yd).mean(-1, keepdim=True) + eps) * weight.double()).to(torch.float32))
        if next_weight is None:
            return None
        return self.rmsnorm(h, next_weight, next_eps, out_dtype)

    def activation(self, u, kind, out_dtype, col0=0, width=None, gate_col=None):
        z = u.double() if width is None else u.double()[:, col0: col0 + width]
        if kind == "gelu_tanh":
            v = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        elif kind == "gelu_erf":
            v = 0.5 * z * (1.0 + torch.erf(z * 0.7071067811865476))
        else:
            v = z * torch.sigmoid(z)
        if gate_col is not None:
            v = v * torch.sigmoid(u.double()[:, gate_col: gate_col + 1])
        return v.to(out_dtype)

    def moe_route(self, logits, correction, experts, top, groups, keep, score="softmax", group_best=1, normalize=False, sum_eps=0.0,
                  scale=1.0, bias=None):
        n = logits.shape[0]
        z = logits.double()[:, :experts] + (bias.double() if bias is not None else 0.0)
        s = torch.softmax(z, dim=-1) if score == "softmax" else torch.sigmoid(z)
        if correction is None:
            correction = torch.zeros(experts)
        dense = torch.zeros(n, experts, dtype=torch.float32)
        ids = torch.zeros(n, top, dtype=torch.int32)
        wts = torch.zeros(n, top, dtype=torch.float32)
        for t in range(n):
            ch = (s[t] + correction.double()).tolist()
            if groups > 1:
                per = experts // groups
                score = [sum(sorted(ch[g * per: (g + 1) * per], reverse=True)[:group_best]) for g in range(groups)]
                kept = sorted(range(groups), key=lambda g: (-score[g], g))[:keep]
                ch = [c if e // per in kept else float("-inf") for e, c in enumerate(ch)]
            order = [e for e in sorted(range(experts), key=lambda e: (-ch[e], e)) if ch[e] != float("-inf")][:top]
            factor = scale / (sum(float(s[t, e]) for e in order) + sum_eps) if normalize else scale
            for i, e in enumerate(order):
                dense[t, e] = s[t, e] * factor
                ids[t, i] = e
                wts[t, i] = s[t, e] * factor
        return dense, ids, wts

    def head_rmsnorm(self, rows, col_a, heads_a, weight_a, col_b, heads_b, weight_b, dim, eps):
        for col, heads, w in ((col_a, heads_a, weight_a), (col_b, heads_b, weight_b)):
            if heads:
                x = rows[:, col: col + heads * dim].double().reshape(rows.shape[0], heads, dim)
                x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.double()
                rows[:, col: col + heads * dim] = x.reshape(rows.shape[0], heads * dim).to(torch.float32)

    def vector_store(self, c, slots, k_cache, v_cache):
        ps = k_cache.shape[2]
        for t in range(c.shape[0]):
            page, off = int(slots[t]) // ps, int(slots[t]) % ps
            k_cache[page, 0, off] = c[t]
            v_cache[page, 0, :, off] = c[t]

    def mlstm_scan(self, proj, col0, i_bias, f_bias, cap, q_scale, state, state_off, cu_seqlens, state_slots, num_requests, heads, dim,
                   vdim, norm_weight, eps, scale, out, out_col0):
        H, D, Dv = heads, dim, vdim
        x = proj.double()[:, col0:]
        cu = cu_seqlens.tolist()
        c_q, c_k, c_v, c_g, c_i, c_f = 0, H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + 2 * H * Dv, 2 * H * D + 2 * H * Dv + H
        n_state = H * (Dv + 1) * D
        for r in range(num_requests):
            slot = int(state_slots[r])
            row = state[slot, state_off: state_off + n_state + H * (Dv + 1)].double()
            S = row[:n_state].reshape(H, Dv + 1, D).clone()      # [head, column, key channel]; the last column is n
            m = row[n_state:].reshape(H, Dv + 1)[:, 0].clone()
            for t in range(cu[r], cu[r + 1]):
                q = x[t, c_q: c_q + H * D].reshape(H, D) * q_scale
                k = x[t, c_k: c_k + H * D].reshape(H, D)
                v = torch.cat([x[t, c_v: c_v + H * Dv].reshape(H, Dv), torch.ones(H, 1, dtype=torch.float64)], dim=1)
                i_log = cap * torch.tanh((x[t, c_i: c_i + H] + i_bias.double()) / cap)
                f_log = torch.nn.functional.logsigmoid(cap * torch.tanh((x[t, c_f: c_f + H] + f_bias.double()) / cap))
                m_new = torch.maximum(f_log + m, i_log)
                S = torch.exp(f_log + m - m_new)[:, None, None] * S + torch.exp(i_log - m_new)[:, None, None] * v[:, :, None] * k[:, None, :]
                m = m_new
                read = torch.einsum("hcd,hd->hc", S, q)
                o = read[:, :Dv] / (torch.maximum(read[:, Dv].abs(), torch.exp(-m)) + 1e-6)[:, None]
                o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
                o = o.reshape(H * Dv) * norm_weight.double() * torch.sigmoid(x[t, c_g: c_g + H * Dv]) * scale
                out[t, out_col0: out_col0 + H * Dv] = o.to(out.dtype)
            state[slot, state_off: state_off + n_state] = S.reshape(-1).to(torch.float32)
            state[slot, state_off + n_state: state_off + n_state + H * (Dv + 1)] = m[:, None].expand(H, Dv + 1).reshape(-1).to(torch.float32)

    def moe_plan(self, ids, experts):
        flat = ids.reshape(-1).tolist()
        counts, rank = [0] * experts, []
        for e in flat:
            rank.append(counts[e])
            counts[e] += 1
        offsets = [0]
        for c in counts:
            offsets.append(offsets[-1] + c)
        return (torch.tensor(counts, dtype=torch.int32), torch.tensor(offsets, dtype=torch.int32),
                torch.tensor(rank, dtype=torch.int32).reshape(ids.shape))

    def moe_gather(self, x, ids, rank, offsets):
        n, top = ids.shape
        row_of = (offsets.long()[ids.long()] + rank.long()).to(torch.int32)
        xg = torch.zeros(n * top, x.shape[1], dtype=x.dtype)
        xg[row_of.long().reshape(-1)] = x.repeat_interleave(top, dim=0)
        return xg, row_of

    def moe_scatter(self, yg, row_of, weights, y=None):
        add = (weights.double()[:, :, None] * yg.double()[row_of.long()]).sum(1)
        if y is None:
            return add.to(torch.float32)
        y.copy_((y.double() + add).to(torch.float32))
        return y

    def moe_spread(self, a, dense, experts):
        n, ff = a.shape[0], a.shape[1] // experts
        return (a.double().reshape(n, experts, ff) * dense.double()[:, :, None]).permute(1, 0, 2).contiguous().to(a.dtype)

    def lowrank_up(self, x, col0, weight_t, mode="plain", a_log=None, bias=None, per_head=0, rate=0.0, in_act=None):
        r = weight_t.shape[0]
        xin = x.double()[:, col0: col0 + r]
        v = (torch.tanh(xin) if in_act == "tanh" else xin) @ weight_t.double()
        if mode == "rate_sigmoid":
            v = torch.exp(-rate * torch.sigmoid(v + bias.double()))
        if mode == "sigmoid":
            v = torch.sigmoid(v)
        elif mode == "decay":
            rate = torch.exp(a_log.double()).repeat_interleave(per_head)
            v = torch.exp(-rate * torch.nn.functional.softplus(v + bias.double()))
        return v.to(torch.float32)

    def delta_scan(self, qkv, decay, proj, beta_col0, state, state_off, cu_seqlens, state_slots, num_requests, heads, kv_heads,
                   dim, vdim, q_scale, unit_eps):
        n = qkv.shape[0]
        rep = heads // kv_heads
        x = qkv.double()
        q = x[:, : kv_heads * dim].reshape(n, kv_heads, dim)
        k = x[:, kv_heads * dim: 2 * kv_heads * dim].reshape(n, kv_heads, dim)
        v = x[:, 2 * kv_heads * dim:].reshape(n, heads, vdim)
        q = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + unit_eps) * q_scale).repeat_interleave(rep, dim=1)
        k = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + unit_eps)).repeat_interleave(rep, dim=1)
        beta = torch.sigmoid(proj.double()[:, beta_col0: beta_col0 + heads])
        g = decay.double().reshape(n, heads, dim)
        y = torch.zeros(n, heads, vdim, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        size = heads * dim * vdim
        for r in range(num_requests):
            if cu[r + 1] <= cu[r]:
                continue
            slot = int(state_slots[r])
            # (in memory a head's state lies column by column: [heads, vdim, dim])
            S = state[slot, state_off: state_off + size].double().reshape(heads, vdim, dim).transpose(1, 2)
            for t in range(cu[r], cu[r + 1]):
                S = g[t][:, :, None] * S
                u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
                S = S + k[t][:, :, None] * u[:, None, :]
                y[t] = torch.einsum("hdv,hd->hv", S, q[t])
            state[slot, state_off: state_off + size] = S.transpose(1, 2).reshape(-1).to(torch.float32)
        return y.reshape(n, heads * vdim).to(torch.float32)

    def head_norm_gate(self, o, weight, gate, eps, scale, heads, out, out_col0, gate_rows=None, gate_col0=0):
        n, vdim = o.shape[0], o.shape[1] // heads
        x = o.double().reshape(n, heads, vdim)
        w = weight.double().reshape(-1, vdim)      # [1, vdim] shared or [heads, vdim]
        x = (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w).reshape(n, heads * vdim)
        if gate is not None:
            x = x * gate.double()
        if gate_rows is not None:
            x = x * torch.sigmoid(gate_rows.double()[:, gate_col0: gate_col0 + heads * vdim])
        out[:, out_col0: out_col0 + heads * vdim] = (x * scale).to(out.dtype)

    def swiglu(self, gu, out_dtype):
        i = gu.shape[1] // 2
        g, u = gu.double()[:, :i], gu.double()[:, i:]
        return (g / (1.0 + torch.exp(-g)) * u).to(out_dtype)

    def argmax(self, logits):
        v = logits.shape[1]
        flipped = torch.flip(logits, dims=[1])
        return (v - 1 - torch.argmax(flipped, dim=1)).to(torch.int32)

    def take_rows(self, t, rows=None):
        return t.clone() if rows is None else t[torch.tensor(list(rows), dtype=torch.long)].clone()

    def zero_rows(self, t, rows):
        if len(rows):
            t[torch.tensor(list(rows), dtype=torch.long)] = 0
