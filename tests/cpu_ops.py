"""A stand-in for the HIP kernel library, in plain torch on the CPU, used only
by tests that check the engine's own logic (batch packing, block tables, cache
manager, run order, scheduler) without a GPU.  The product never loads this:
its kernel library is tiny_llm_infer_amd.kernels.ops.HipOps and nothing else.
"""
from __future__ import annotations

import torch


class CpuOps:
    name = "cpu-test-double"

    def check_attention_sizes(self, heads, kv_heads, head_dim):
        pass

    def check_page_size(self, page_size):
        pass

    def feed_tokens(self, token_ids, token_from, src, rows):
        take = token_from[:rows] >= 0
        token_ids[:rows][take] = src[token_from[:rows][take].long()]

    def embed(self, table, token_ids, num_rows, scale=1.0, positions=None, pos_table=None):
        x = table[token_ids[:num_rows].long()].to(torch.float32) * scale
        if pos_table is not None:
            x = x + pos_table[positions[:num_rows].long()].to(torch.float32)
        return x

    def softcap(self, logits, cap):
        return cap * torch.tanh(logits / cap)

    def check_activation(self, name):
        assert name in ("relu2", "relu", "silu", "gelu_tanh")

    def activation(self, x, name):
        z = x.to(torch.float32)
        if name == "relu2":
            y = torch.relu(z) ** 2
        elif name == "relu":
            y = torch.relu(z)
        elif name == "silu":
            y = z / (1 + torch.exp(-z))
        else:
            y = 0.5 * z * (1 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        return y.to(x.dtype)

    # ---- several residual streams ------------------------------------------------
    def check_streams(self, streams, width):
        pass

    def streams_open(self, x, streams):
        return x[:, None, :].repeat(1, streams, 1).contiguous()

    def streams_norm(self, resid, pending, w_in, weight, eps, out_dtype, rows=None, num_rows=None, shift=None):
        x = resid
        if pending is not None:
            y = self.resolve(pending.y).to(torch.float32)
            x = torch.einsum("st,rsd->rtd", pending.mix, resid) + pending.out[None, :, None] * y[:, None, :]
            if rows is None:
                resid.copy_(x)
        if rows is not None:
            x = x[rows[:num_rows].long()]
        u = torch.einsum("s,rsd->rd", w_in, x)
        h = weight * u * torch.rsqrt((u * u).mean(dim=-1, keepdim=True) + eps)
        if shift is None:
            return h.to(out_dtype)
        mu, state, step = shift
        return self.token_shift(h, mu, state, step, out_dtype)

    def token_shift(self, h, mu, state, step, out_dtype):
        out = torch.empty_like(h)
        for i in range(step.num_seqs):
            r0, r1 = step.h_row_start[i], step.h_row_start[i + 1]
            slot = step.h_slots[i]
            first = state[slot].clone() if step.h_seq_start[i] > 0 else torch.zeros_like(state[slot])
            prev = torch.cat([first[None], h[r0:r1 - 1]], dim=0)
            out[r0:r1] = h[r0:r1] + (prev - h[r0:r1]) * mu
            state[slot] = h[r1 - 1]
        return out.to(out_dtype)

    # ---- attention with convolved queries and keys, values = keys ----------------------
    def check_conv_attention_sizes(self, heads, kv_heads, head_dim, taps):
        pass

    def conv_key_attention(self, qk, bias, conv, state, step, cache, heads, kv_heads, head_dim, taps, scale,
                           temp, penalty, mask):
        T = step.num_rows
        qd = heads * head_dim
        raw = qk.to(torch.float32)
        mixed = torch.empty_like(raw)
        for i in range(step.num_seqs):
            r0, r1 = step.h_row_start[i], step.h_row_start[i + 1]
            slot, start = step.h_slots[i], step.h_seq_start[i]
            if taps > 1:
                before = state[slot].to(torch.float32).clone()
                known = torch.arange(start - taps + 1, start) >= 0          # positions before 0 hold nothing
                hist = torch.where(known[:, None], before + bias, torch.zeros_like(before))
                u = torch.cat([hist, raw[r0:r1] + bias], dim=0)
                state[slot] = torch.cat([before, raw[r0:r1]], dim=0)[-(taps - 1):].to(state.dtype)
            else:
                u = raw[r0:r1] + bias
            n = r1 - r0
            mixed[r0:r1] = sum(conv[j] * u[j:j + n] for j in range(taps))          # conv: [taps, channels]
        q = mixed[:, :qd].to(qk.dtype).to(torch.float32).reshape(T, heads, head_dim)
        k = mixed[:, qd:].reshape(T, kv_heads, head_dim)
        page = cache.group.page_size
        tables = cache.group.tables
        pos = step.positions[:T].long()
        seq = step.seq_of_row[:T].long()
        pages = tables[seq, pos // page].long()
        assert (pages >= 0).all(), "a row writes to a page that is not held"
        cache.record("k")[pages, :, pos % page] = k.to(cache.record("k").dtype)
        out = torch.zeros(T, heads, head_dim)
        mul = heads // kv_heads
        for r in range(T):
            p = int(pos[r])
            lo = 0
            if mask is not None:
                lo = p // mask[1] * mask[1] if mask[0] == "chunk" else max(0, p - mask[1] + 1)
            idx = torch.arange(lo, p + 1)
            pg = tables[int(seq[r]), idx // page].long()
            assert (pg >= 0).all(), "a row reads a page that is not held"
            kk = cache.record("k")[pg, :, idx % page].to(torch.float32)          # [n, kv, d]
            dist = (p - idx).to(torch.float32)
            for h in range(heads):
                s = (kk[:, h // mul] @ q[r, h]) * scale
                if temp is not None:
                    s = s * temp[h]
                if penalty is not None:
                    s = s - penalty[0][h] * torch.log(1.0 + penalty[1][h] * dist)
                out[r, h] = torch.softmax(s, dim=0) @ kk[:, h // mul]
        return out.reshape(T, qd).to(qk.dtype)

    # ---- layer norm, the gated delta rule, routed experts ---------------------------------
    def add_layernorm(self, resid, deltas, weights, eps, out_dtype, rows=None, num_rows=None):
        owed = None
        for d in deltas:
            owed = d.to(torch.float32) if owed is None else owed + d.to(torch.float32)
        if rows is None:
            if owed is not None:
                resid += owed
            x = resid
        else:
            x = resid[rows[:num_rows].long()]
            if owed is not None:
                x = x + owed[rows[:num_rows].long()]
        m = x.mean(dim=-1, keepdim=True)
        z = (x - m) * torch.rsqrt(((x - m) ** 2).mean(dim=-1, keepdim=True) + eps)
        return [(z * w).to(out_dtype) for w in weights]

    def check_delta_sizes(self, heads, kv_heads, dk, dv, taps):
        pass

    def small_product(self, x, w_rows):
        return x.to(torch.float32) @ w_rows.to(torch.float32).t(), False

    def delta_state_shape(self, heads, dk, dv):
        return (heads, dk, dv)

    def delta_rule(self, proj, gates, conv, a_log, dt_bias, kept, state, step, heads, kv_heads, dk, dv, taps,
                   gates_transposed=False):
        T = step.num_rows
        gates = gates.t() if gates_transposed else gates
        qd, vd = kv_heads * dk, heads * dv
        C = 2 * qd + vd
        raw = proj[:, :C].to(torch.float32)
        out = torch.zeros(T, heads, dv)
        rep = heads // kv_heads
        for i in range(step.num_seqs):
            r0, r1 = step.h_row_start[i], step.h_row_start[i + 1]
            slot, start, n = step.h_slots[i], step.h_seq_start[i], step.h_row_start[i + 1] - step.h_row_start[i]
            hist = torch.zeros(taps - 1, C)
            if taps > 1 and start > 0:
                hist = kept[slot].to(torch.float32).clone()
                hist[torch.arange(start - taps + 1, start) < 0] = 0.0
            u = torch.cat([hist, raw[r0:r1]], dim=0)
            if taps > 1:
                kept[slot] = u[-(taps - 1):].to(kept.dtype)
            c = sum(conv[j] * u[j:j + n] for j in range(taps))
            c = c / (1 + torch.exp(-c))
            q = c[:, :qd].reshape(n, kv_heads, dk)
            k = c[:, qd:2 * qd].reshape(n, kv_heads, dk)
            v = c[:, 2 * qd:].reshape(n, heads, dv)
            q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
            k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
            beta = torch.sigmoid(gates[r0:r1, :heads])
            decay = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(gates[r0:r1, heads:] + dt_bias))
            S = state[slot].clone() if start > 0 else torch.zeros(heads, dk, dv)
            for t in range(n):
                kk, qq = k[t].repeat_interleave(rep, 0), q[t].repeat_interleave(rep, 0)      # [H, dk]
                S = S * decay[t][:, None, None]
                uu = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, kk))
                S = S + kk[:, :, None] * uu[:, None, :]
                out[r0 + t] = torch.einsum("hkv,hk->hv", S, qq)
            state[slot] = S
        return out.reshape(T, vd)

    def gated_rmsnorm(self, o, proj, gate_at, weight, eps, heads, dv, out_dtype):
        T = o.shape[0]
        x = o.reshape(T, heads, dv)
        g = proj[:, gate_at:gate_at + heads * dv].to(torch.float32).reshape(T, heads, dv)
        y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * weight * (g / (1 + torch.exp(-g)))
        return y.reshape(T, heads * dv).to(out_dtype)

    def check_expert_sizes(self, experts, top, groups, keep, hidden, inter):
        pass

    def pack_experts(self, w_gate_up, w_down):
        return None

    def check_router(self, score, group_score):
        assert score in ("sigmoid", "softmax") and group_score in ("top2", "max")

    def route_experts(self, z, experts, top, groups, keep, scale, has_shared, transposed=False, score="sigmoid",
                      group_score="top2", normalize=True, correction=None):
        z = z.t() if transposed else z
        T = z.shape[0]
        s = torch.sigmoid(z[:, :experts]) if score == "sigmoid" else torch.softmax(z[:, :experts], dim=-1)
        c = s if correction is None else s + correction
        per = experts // groups
        by_group = c.reshape(T, groups, per)
        group = by_group.topk(min(2, per), dim=-1).values.sum(-1) if group_score == "top2" else by_group.max(-1).values
        best = group.topk(keep, dim=-1).indices
        open_ = torch.zeros(T, groups, dtype=torch.bool)
        open_.scatter_(1, best, True)
        masked = torch.where(open_.repeat_interleave(per, 1), c, torch.full_like(c, float("-inf")))
        ids = masked.topk(top, dim=-1).indices
        w = s.gather(1, ids)
        w = w / (w.sum(-1, keepdim=True) + 1e-20) * scale if normalize else w * scale
        return ids.to(torch.int32), w, (torch.sigmoid(z[:, experts]) if has_shared else None)

    def apply_experts(self, x, ids, weights, w_gate_up, w_down, packed, shared, shared_gate, limit=0.0, slope=1.0):
        T, n = x.shape
        E = w_gate_up.shape[0]
        ff = w_gate_up.shape[1] // 2
        xf = x.to(torch.float32)
        out = torch.zeros(T, n)
        for t in range(T):
            for j in range(ids.shape[1]):
                e = int(ids[t, j])
                if e >= E:                          # an expert that hands its input on
                    out[t] += weights[t, j] * xf[t]
                    continue
                gu = w_gate_up[e].to(torch.float32) @ xf[t]
                a = self._gated(gu[:ff], gu[ff:], limit, slope).to(x.dtype).to(torch.float32)
                out[t] += weights[t, j] * (w_down[e].to(torch.float32) @ a)
        if shared is not None:
            out = out + (shared.to(torch.float32) if shared_gate is None else shared_gate[:, None] * shared.to(torch.float32))
        return out.to(x.dtype)

    # ---- blocks that norm what a sublayer gives; attention with sizes of its own ----
    def residual_rows(self, resid, dtype):
        return resid if dtype == torch.float32 else resid.to(dtype)

    def norm_add(self, resid, y, weight, eps, out_dtype):
        yf = y.to(torch.float32)
        resid += weight * yf * torch.rsqrt((yf * yf).mean(dim=-1, keepdim=True) + eps)
        return resid if out_dtype == torch.float32 else resid.to(out_dtype)

    def check_sized_attention(self, heads, kv_heads, key_dim, value_dim):
        pass

    @staticmethod
    def _seen(p, window, keep_first):
        """The positions a row at p sees, ascending."""
        if not window:
            return torch.arange(0, p + 1)
        lo = max(0, p - window + 1)
        return torch.cat([torch.arange(0, min(keep_first, lo)), torch.arange(lo, p + 1)])

    def differential_attention(self, proj, step, cache, heads, kv_heads, dim, vdim, q_weight, k_weight, norm_eps, scale,
                               lam, after, window, keep_first):
        T = step.num_rows
        x = proj.to(torch.float32)
        nq, nk, nv = heads * 2 * dim, kv_heads * 2 * dim, kv_heads * vdim

        def norm(t, w):
            return w * t * torch.rsqrt((t * t).mean(dim=-1, keepdim=True) + norm_eps)
        q = norm(x[:, :nq].reshape(T, heads * 2, dim), q_weight).to(proj.dtype).to(torch.float32)
        k = norm(x[:, nq:nq + nk].reshape(T, kv_heads * 2, dim), k_weight)
        v = x[:, nq + nk:nq + nk + nv].reshape(T, kv_heads, vdim)
        gate = torch.sigmoid(x[:, nq + nk + nv:])
        page, tables = cache.group.page_size, cache.group.tables
        pos, seq = step.positions.long(), step.seq_of_row.long()
        pages = tables[seq, pos // page].long()
        assert (pages >= 0).all(), "a row writes to a page that is not held"
        kc, vc = cache.record("k"), cache.record("v")
        kc[pages, :, pos % page] = k.to(kc.dtype)
        vc[pages, :, :, pos % page] = v.to(vc.dtype)
        out = torch.zeros(T, heads, vdim)
        mul = heads // kv_heads
        for r in range(T):
            idx = self._seen(int(pos[r]), window, keep_first)
            pg = tables[int(seq[r]), idx // page].long()
            assert (pg >= 0).all(), "a row reads a page that is not held"
            kk = kc[pg, :, idx % page].to(torch.float32)            # [n, kv * 2, dim]
            vv = vc[pg, :, :, idx % page].to(torch.float32)         # [n, kv, vdim]
            for h in range(heads):
                g = h // mul
                a = [torch.softmax((kk[:, g * 2 + m] @ q[r, h * 2 + m]) * scale, dim=0) @ vv[:, g] for m in range(2)]
                o = a[0] - lam * a[1]
                out[r, h] = o * torch.rsqrt((o * o).mean() + norm_eps) * after * gate[r, h]
        return out.reshape(T, heads * vdim).to(proj.dtype)

    def latent_attention(self, proj, step, cache, heads, dim, rot, rank, vdim, norm_weight, norm_eps, rotary, scale,
                         w_qk, w_v, sinks=None):
        T = step.num_rows
        x = proj.to(torch.float32)
        cos, sin, rd = rotary
        half = rd // 2
        pos, seq = step.positions.long(), step.seq_of_row.long()

        def turn(t, c, s):
            a, b, rest = t[..., :half], t[..., half:rd], t[..., rd:]
            return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)
        q = x[:, :heads * (dim + rot)].reshape(T, heads, dim + rot)
        down = x[:, heads * (dim + rot):]
        c = down[:, :rank]
        c = norm_weight * c * torch.rsqrt((c * c).mean(dim=-1, keepdim=True) + norm_eps)
        entry = torch.cat([c, turn(down[:, rank:], cos[pos], sin[pos])], dim=-1)
        page, tables = cache.group.page_size, cache.group.tables
        pages = tables[seq, pos // page].long()
        assert (pages >= 0).all(), "a row writes to a page that is not held"
        kc = cache.record("latent")
        kc[pages, pos % page] = entry.to(kc.dtype)
        q_lat = torch.einsum("thd,hnd->thn", q[..., :dim].to(proj.dtype).to(torch.float32), w_qk.to(torch.float32))
        qk = torch.cat([q_lat, turn(q[..., dim:], cos[pos][:, None], sin[pos][:, None])], dim=-1).to(proj.dtype).to(torch.float32)
        o = torch.zeros(T, heads, rank)
        for r in range(T):
            idx = torch.arange(0, int(pos[r]) + 1)
            pg = tables[int(seq[r]), idx // page].long()
            assert (pg >= 0).all(), "a row reads a page that is not held"
            kk = kc[pg, idx % page].to(torch.float32)               # [n, rank + rot]
            sc = (qk[r] @ kk.t()) * scale                           # [heads, n]
            if sinks is not None:
                sc = torch.cat([sc, sinks[:, None]], dim=-1)
            w = torch.softmax(sc, dim=-1)[:, :len(idx)]
            o[r] = w @ kk[:, :rank]
        o = o.to(proj.dtype).to(torch.float32)
        return torch.einsum("thn,hen->the", o, w_v.to(torch.float32)).reshape(T, heads * vdim).to(proj.dtype)

    def add_rmsnorm(self, resid, delta, weight, eps, out_dtype, rows=None, num_rows=None, lazy=False):
        if rows is None:
            if delta is not None:
                resid += delta.to(torch.float32)
            x = resid
        else:
            x = resid[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].to(torch.float32)
        scale = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
        return (weight * x * scale).to(out_dtype)

    def resolve(self, y):
        return y

    def linear(self, x, w, out_dtype=None, deferred=False, sums_only=False):
        w = getattr(w, "w", w)
        y = x.to(torch.float32) @ w.to(torch.float32).t()
        return y.to(out_dtype or x.dtype)

    def linear_swiglu(self, x, m):
        return self.swiglu(self.linear(x, m))

    @staticmethod
    def _gated(g, u, limit, slope):
        if limit <= 0:
            return g / (1 + torch.exp(-g)) * u
        g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
        return g / (1 + torch.exp(-slope * g)) * (u + 1)

    def swiglu(self, gu, limit=0.0, slope=1.0):
        inter = gu.shape[1] // 2
        g, u = gu[:, :inter].to(torch.float32), gu[:, inter:].to(torch.float32)
        return self._gated(g, u, limit, slope).to(gu.dtype)

    # ---- attention with biases and a sink whose values may be its keys; lightning attention ----
    def sink_attention(self, proj, step, cache, heads, kv_heads, head_dim, bias, rotary, scale, sinks, window,
                       values_are_keys):
        T = step.num_rows
        qd, kd = heads * head_dim, kv_heads * head_dim
        x = proj.to(torch.float32)
        if bias is not None:
            x = x + bias
        q = x[:, :qd].reshape(T, heads, head_dim)
        k = x[:, qd:qd + kd].reshape(T, kv_heads, head_dim)
        v = k if values_are_keys else x[:, qd + kd:].reshape(T, kv_heads, head_dim)
        pos, seq = step.positions.long(), step.seq_of_row.long()
        if rotary is not None:
            cos, sin, rd = rotary
            half = rd // 2
            c, s_ = cos[pos][:, None, :], sin[pos][:, None, :]

            def rot(t):
                a, b, rest = t[..., :half], t[..., half:rd], t[..., rd:]
                return torch.cat([a * c - b * s_, b * c + a * s_, rest], dim=-1)
            q, k = rot(q), rot(k)
        page, tables = cache.group.page_size, cache.group.tables
        pages = tables[seq, pos // page].long()
        assert (pages >= 0).all(), "a row writes to a page that is not held"
        kc, vc = cache.record("k"), cache.record("v")
        kc[pages, :, pos % page] = k.to(kc.dtype)
        vc[pages, :, :, pos % page] = v.to(vc.dtype)
        q = q.to(proj.dtype).to(torch.float32)
        out = torch.zeros(T, heads, head_dim)
        mul = heads // kv_heads
        for r in range(T):
            idx = self._seen(int(pos[r]), window, 0)
            pg = tables[int(seq[r]), idx // page].long()
            assert (pg >= 0).all(), "a row reads a page that is not held"
            kk = kc[pg, :, idx % page].to(torch.float32)            # [n, kv, d]
            vv = vc[pg, :, :, idx % page].to(torch.float32)
            for h in range(heads):
                sc = (kk[:, h // mul] @ q[r, h]) * scale
                if sinks is not None:
                    sc = torch.cat([sc, sinks[h:h + 1]])
                w = torch.softmax(sc, dim=0)[:len(idx)]
                out[r, h] = w @ vv[:, h // mul]
        return out.reshape(T, qd).to(proj.dtype)

    def add_bias(self, y, bias):
        return (y.to(torch.float32) + bias).to(y.dtype)

    def check_lightning_sizes(self, heads, dk, dv):
        pass

    def lightning_state_shape(self, heads, dk, dv):
        return (heads, dv, dk)

    def lightning_attention(self, proj, decay, state, step, heads, dk, dv):
        T = step.num_rows
        x = proj.to(torch.float32)
        x = x / (1 + torch.exp(-x))
        q = x[:, :heads * dk].reshape(T, heads, dk)
        k = x[:, heads * dk:2 * heads * dk].reshape(T, heads, dk)
        v = x[:, 2 * heads * dk:2 * heads * dk + heads * dv].reshape(T, heads, dv)
        out = torch.zeros(T, heads, dv)
        for i in range(step.num_seqs):
            r0, r1 = step.h_row_start[i], step.h_row_start[i + 1]
            slot = step.h_slots[i]
            S = state[slot].clone() if step.h_seq_start[i] > 0 else torch.zeros(heads, dv, dk)      # [H, dv, dk]
            for t in range(r0, r1):
                S = decay[:, None, None] * S + v[t][:, :, None] * k[t][:, None, :]
                out[t] = torch.einsum("hvk,hk->hv", S, q[t])
            state[slot] = S
        return out.reshape(T, heads * dv)

    def lightning_norm(self, o, proj, gate_at, weight, eps, out_dtype):
        n = o.shape[1]
        g = proj[:, gate_at:gate_at + n].to(torch.float32)
        return (o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * weight * torch.sigmoid(g)).to(out_dtype)

    def qkv_to_cache(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary):
        T = step.num_rows
        qd, kd = heads * head_dim, kv_heads * head_dim
        x = qkv.to(torch.float32)
        q = x[:, :qd].reshape(T, heads, head_dim)
        k = x[:, qd:qd + kd].reshape(T, kv_heads, head_dim)
        v = x[:, qd + kd:].reshape(T, kv_heads, head_dim)

        def norm(t, wn):
            if wn is None:
                return t
            w, eps = wn
            return w * t * torch.rsqrt((t * t).mean(dim=-1, keepdim=True) + eps)

        q, k = norm(q, q_norm), norm(k, k_norm)
        pos = step.positions.long()
        if rotary is not None:
            cos, sin, rd = rotary
            half = rd // 2
            c, s = cos[pos][:, None, :], sin[pos][:, None, :]

            def rot(t):
                a, b, rest = t[..., :half], t[..., half:rd], t[..., rd:]
                return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)
            q, k = rot(q), rot(k)
        if cache is not None and cache.writes:
            page = cache.group.page_size
            tables = cache.group.tables
            seq = step.seq_of_row.long()
            pages = tables[seq, pos // page].long()
            assert (pages >= 0).all(), "a row writes to a page that is not held"
            slots = pos % page
            cache.record("k")[pages, :, slots] = k.to(cache.record("k").dtype)
            cache.record("v")[pages, :, :, slots] = v.to(cache.record("v").dtype)        # values are kept transposed
        return q.reshape(T, qd).to(qkv.dtype)

    def qkv_attention(self, qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary, scale, window):
        q = self.qkv_to_cache(qkv, step, cache, heads, kv_heads, head_dim, q_norm, k_norm, rotary)
        return self.paged_attention(q, step, cache, heads, kv_heads, head_dim, scale, window)

    def paged_attention(self, q, step, cache, heads, kv_heads, head_dim, scale, window):
        T = step.num_rows
        page = cache.group.page_size
        tables = cache.group.tables
        qf = q.to(torch.float32).reshape(T, heads, head_dim)
        out = torch.zeros(T, heads, head_dim, dtype=torch.float32)
        mul = heads // kv_heads
        pos_l = step.positions.tolist()
        seq_l = step.seq_of_row.tolist()
        for r in range(T):
            p = pos_l[r]
            lo = 0 if window is None else max(0, p - window + 1)
            idx = torch.arange(lo, p + 1)
            pages = tables[seq_l[r], idx // page].long()
            assert (pages >= 0).all(), "a row reads a page that is not held"
            kk = cache.record("k")[pages, :, idx % page].to(torch.float32)     # [n, kv, d]
            vv = cache.record("v")[pages, :, :, idx % page].to(torch.float32)
            for h in range(heads):
                s = (kk[:, h // mul] @ qf[r, h]) * scale
                w = torch.softmax(s, dim=0)
                out[r, h] = w @ vv[:, h // mul]
        return out.reshape(T, heads * head_dim).to(q.dtype)

    # ---- sampling: the same hash and rule as csrc/sampling.hip, in Python ----
    @staticmethod
    def _mix32(h):
        h &= 0xFFFFFFFF
        h ^= h >> 16
        h = (h * 0x85EBCA6B) & 0xFFFFFFFF
        h ^= h >> 13
        h = (h * 0xC2B2AE35) & 0xFFFFFFFF
        h ^= h >> 16
        return h

    @classmethod
    def uniform(cls, seed, token):
        seed &= (1 << 64) - 1
        lo, hi = seed & 0xFFFFFFFF, seed >> 32
        h = cls._mix32(token ^ 0x9E3779B9)
        h = cls._mix32(h ^ lo)
        h = cls._mix32((h + hi * 0x85EBCA6B + 0x27D4EB2F) & 0xFFFFFFFF)
        return ((h >> 9) + 0.5) / 8388608.0

    def sample(self, logits, temperatures=None, seeds=None, top_p=None):
        import math
        out = []
        for r in range(logits.shape[0]):
            row = logits[r].double()
            temp = 0.0 if temperatures is None else float(temperatures[r])
            if temp <= 1e-6:
                out.append(int(torch.argmax(row)))
                continue
            keep = torch.ones_like(row, dtype=torch.bool)
            if top_p is not None and float(top_p[r]) < 1.0:
                w = torch.exp((row - row.max()) / temp)
                order = torch.argsort(w, descending=True)
                csum = torch.cumsum(w[order], 0)
                n = int((csum < float(top_p[r]) * w.sum()).sum()) + 1
                keep[:] = False
                keep[order[:n]] = True
            seed = int(seeds[r])
            g = torch.tensor([-math.log(-math.log(self.uniform(seed, t))) for t in range(row.numel())],
                             dtype=torch.float64)
            score = torch.where(keep, row + temp * g, torch.full_like(row, -float("inf")))
            out.append(int(torch.argmax(score)))
        return torch.tensor(out, dtype=torch.int32)
