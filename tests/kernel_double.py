"""A CPU stand-in for the kernel library, for tests of the engine's bookkeeping.

It has the method names and argument meaning of ``reinfer_amd.kernels.ops.HipKernels``
and computes with torch on the CPU, reading and writing the same paged cache
through the same index arrays. With it the ``not gpu`` tests can run the step
function, the cache manager and the scheduler end to end where there is no GPU.
It is not part of the product and nothing in ``reinfer_amd`` imports it; on a GPU
box the tests use the real kernels.
"""
from __future__ import annotations

import torch

from reinfer_amd.cache.layout import unpack_k, unpack_v


def k_index(off, e, d):
    """Element (slot off, e) of a (block, KV head) slab, as csrc/common.h cache_k_index."""
    return (off >> 4) * 16 * d + ((e >> 3) * 16 + (off & 15)) * 8 + (e & 7)


def v_index(off, e, d):
    s = off & 15
    return (off >> 4) * 16 * d + (((e >> 4) * 4 + (s >> 2)) * 16 + (e & 15)) * 4 + (s & 3)


class KernelDouble:
    name = "cpu-double"

    def embed(self, table, ids, out, scale=1.0):
        out.copy_(table[ids.long()].float() * scale)

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None, delta_scale=1.0, groups=1):
        if rows is None:
            if delta is not None:
                resid.add_(delta.float() * delta_scale)
            x = resid
        else:
            x = resid[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].float() * delta_scale
        n, h = x.shape
        xg = x.view(n, groups, h // groups)
        rstd = torch.rsqrt((xg * xg).mean(dim=-1, keepdim=True) + eps)
        out.copy_(((xg * rstd).reshape(n, h) * weight.float()).to(out.dtype))

    def qk_norm_rope_cache(self, qkv, q_weight, k_weight, eps, positions, inv_freq, rotary_dim,
                           rope_style, slots, kcache, vcache, num_heads, num_kv_heads, head_dim):
        T = qkv.shape[0]
        d = head_dim
        u = qkv.view(T, num_heads + 2 * num_kv_heads, d).float()
        q, k, v = u[:, :num_heads], u[:, num_heads:num_heads + num_kv_heads], u[:, num_heads + num_kv_heads:]

        def norm(x, w):
            if w is None:
                return x
            return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w.float()

        def rot(x):
            if rotary_dim == 0:
                return x
            half = rotary_dim // 2
            ang = positions.float()[:, None] * inv_freq[:half].float()[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            out = x.clone()
            if rope_style == 0:
                a, b = x[..., :half], x[..., half:rotary_dim]
                out[..., :half] = a * c - b * s
                out[..., half:rotary_dim] = a * s + b * c
            else:
                a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
                out[..., 0:rotary_dim:2] = a * c - b * s
                out[..., 1:rotary_dim:2] = a * s + b * c
            return out

        q = rot(norm(q, q_weight))
        k = rot(norm(k, k_weight))
        qkv.view(T, -1, d)[:, :num_heads] = q.to(qkv.dtype)
        bs = kcache.shape[2] * 16
        kflat, vflat = kcache.view(kcache.shape[0], num_kv_heads, -1), vcache.view(vcache.shape[0], num_kv_heads, -1)
        e = torch.arange(d)
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            kflat[s // bs][:, k_index(s % bs, e, d)] = k[t].to(kcache.dtype)
            vflat[s // bs][:, v_index(s % bs, e, d)] = v[t].to(vcache.dtype)

    # ---- around the stream
    def pair_hash_add(self, resid, table, batch, last_token, buckets, mul_prev, mul_cur):
        ids, pos = batch.token_ids.tolist(), batch.positions.tolist()
        cu, seq_of = batch.cu_tokens.tolist(), batch.seq_of_token.tolist()
        for t in range(batch.num_tokens):
            i = seq_of[t]
            slot = int(batch.state_slots[i])
            prev = -1
            if t != cu[i]:
                prev = ids[t - 1]
            else:
                if pos[t] > 0 and slot >= 0:
                    prev = int(last_token[slot])
                if slot >= 0:
                    last_token[slot] = ids[cu[i + 1] - 1]
            row = buckets if (pos[t] == 0 or prev < 0) else (prev * mul_prev + ids[t] * mul_cur) % buckets
            resid[t] += table[row].float()

    def stream_add(self, resid, delta=None, other=None, vec=None, delta_scale=1.0):
        if delta is not None:
            resid.add_(delta.float() * delta_scale)
        if other is not None:
            resid.add_(other)
        if vec is not None:
            resid.add_(vec.float())

    def tanh_cap(self, logits, cap):
        logits.copy_(cap * torch.tanh(logits / cap))

    # ---- latent attention
    def latent_prep(self, proj, q_off, dkv_off, c_weight, eps, positions, inv_freq, rot_dims, rot_width, rank,
                    num_heads, head_dim, q_lat, slots, kcache, vcache):
        T = proj.shape[0]
        Dp = q_lat.shape[2]
        half = rot_dims // 2
        ang = positions.float()[:, None] * inv_freq[:half].float()[None, :] if half else None

        def rot(x):                      # [T, ..., rot_width]
            if not half:
                return x
            shape = [T] + [1] * (x.dim() - 2) + [half]
            c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
            out = x.clone()
            a, b = x[..., :half], x[..., half:rot_dims]
            out[..., :half] = a * c - b * s
            out[..., half:rot_dims] = b * c + a * s
            return out

        p = proj.float()
        craw = p[:, dkv_off:dkv_off + rank]
        c = craw * torch.rsqrt((craw * craw).mean(dim=-1, keepdim=True) + eps) * c_weight.float()
        kr = rot(p[:, dkv_off + rank:dkv_off + rank + rot_width])
        row = torch.zeros((T, Dp))
        row[:, :rank] = c
        row[:, rank:rank + rot_width] = kr
        q = p[:, q_off:q_off + num_heads * (head_dim + rot_width)].view(T, num_heads, head_dim + rot_width)
        q_lat[:, :, rank:] = 0
        q_lat[:, :, rank:rank + rot_width] = rot(q[:, :, head_dim:]).to(q_lat.dtype)
        bs = kcache.shape[2] * 16
        kflat, vflat = kcache.view(kcache.shape[0], 1, -1), vcache.view(vcache.shape[0], 1, -1)
        e = torch.arange(Dp)
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            kflat[s // bs][:, k_index(s % bs, e, Dp)] = row[t].to(kcache.dtype)
            vflat[s // bs][:, v_index(s % bs, e, Dp)] = row[t].to(vcache.dtype)

    def head_linear(self, x, x_head, weight, out, o_head, gate=None, gate_per_head=False):
        H, N, K = weight.shape
        for h in range(H):
            y = x[:, h * x_head:h * x_head + K].float() @ weight[h].float().T
            if gate is not None:
                y = y * torch.sigmoid((gate[:, h:h + 1] if gate_per_head else gate[:, h * N:(h + 1) * N]).float())
            out[:, h * o_head:h * o_head + N] = y.to(out.dtype)

    # ---- recurrent mixers (state in a layout of this stand-in's own: the state is the kernels' private matter)
    @staticmethod
    def scan_state_floats(kind, heads, key_dim, value_dim):
        return heads * key_dim * value_dim + (heads * (key_dim + 1) if kind == "matrix_memory" else 0)   # the others: S alone

    @staticmethod
    def _requests(batch):
        """(first row, rows, state slot, fresh) of every request of the step."""
        cu, slots, fresh = batch.cu_tokens.tolist(), batch.state_slots.tolist(), batch.fresh.tolist()
        return [(cu[i], cu[i + 1] - cu[i], slots[i], bool(fresh[i])) for i in range(batch.num_seqs)]

    def matrix_memory_scan(self, proj, q_off, k_off, v_off, gates, gate_bias, state, batch, H, dk, dv, cap, q_scale,
                           denom_eps, out):
        p = proj.float()
        z = gates + gate_bias
        if cap > 0:
            z = cap * torch.tanh(z / cap)
        a_in, b_f = z[:, :H], torch.nn.functional.logsigmoid(z[:, H:])
        nS = H * dk * dv
        for first, rows, slot, fresh in self._requests(batch):
            if slot < 0:
                out[first:first + rows] = 0
                continue
            st = state[slot]
            if fresh:
                st.zero_()
            S, n, m = st[:nS].view(H, dk, dv), st[nS:nS + H * dk].view(H, dk), st[nS + H * dk:]
            for t in range(first, first + rows):
                q = p[t, q_off:q_off + H * dk].view(H, dk) * q_scale
                k = p[t, k_off:k_off + H * dk].view(H, dk)
                v = p[t, v_off:v_off + H * dv].view(H, dv)
                m_new = torch.maximum(b_f[t] + m, a_in[t])
                keep, take = torch.exp(b_f[t] + m - m_new), torch.exp(a_in[t] - m_new)
                S.mul_(keep[:, None, None]).add_(take[:, None, None] * k[:, :, None] * v[:, None, :])
                n.mul_(keep[:, None]).add_(take[:, None] * k)
                m.copy_(m_new)
                den = torch.maximum((n * q).sum(-1).abs(), torch.exp(-m)) + denom_eps
                out[t] = (torch.einsum("hkv,hk->hv", S, q) / den[:, None]).reshape(-1)

    def head_norm_gate(self, read, weight, per_head, gate, kind, eps, H, dv, out):
        T = read.shape[0]
        o = read.view(T, H, dv)
        o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps)
        o = o * (weight.view(H, dv) if per_head else weight.view(1, dv))
        g = gate[:, :H * dv].float().view(T, H, dv)
        g = torch.sigmoid(g) if kind == "sigmoid" else g * torch.sigmoid(g)
        out.copy_((o * g).reshape(T, H * dv).to(out.dtype))

    def delta_rule_prepare(self, proj, filt, state, conv_off, batch, G, dk, H, dv, taps, unit_eps, q_scale, qkv):
        C = 2 * G * dk + H * dv
        x = proj[:, :C].float()
        for first, rows, slot, fresh in self._requests(batch):
            if slot < 0:
                qkv[first:first + rows] = 0
                continue
            tail = state[slot, conv_off:conv_off + (taps - 1) * C].view(taps - 1, C)
            if fresh:
                tail.zero_()
            seq = torch.cat([tail, x[first:first + rows]], dim=0)
            y = sum(seq[j:j + rows] * filt[:, j][None, :] for j in range(taps))
            y = y * torch.sigmoid(y)
            q, k = y[:, :G * dk].reshape(rows, G, dk), y[:, G * dk:2 * G * dk].reshape(rows, G, dk)
            q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + unit_eps) * q_scale
            k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + unit_eps)
            qkv[first:first + rows] = torch.cat([q.reshape(rows, -1), k.reshape(rows, -1), y[:, 2 * G * dk:]], dim=1)
            if taps > 1:
                tail.copy_(seq[rows:].clone())

    def delta_rule_scan(self, qkv, ba, a_log, dt_bias, state, batch, H, G, dk, dv, out):
        beta = torch.sigmoid(ba[:, :H])
        decay = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(ba[:, H:] + dt_bias))
        rep = H // G
        for first, rows, slot, fresh in self._requests(batch):
            if slot < 0:
                out[first:first + rows] = 0
                continue
            S = state[slot, :H * dk * dv].view(H, dk, dv)
            if fresh:
                S.zero_()
            for t in range(first, first + rows):
                q = qkv[t, :G * dk].view(G, dk).repeat_interleave(rep, 0)
                k = qkv[t, G * dk:2 * G * dk].view(G, dk).repeat_interleave(rep, 0)
                v = qkv[t, 2 * G * dk:].view(H, dv)
                S.mul_(decay[t][:, None, None])
                u = beta[t][:, None] * (v - torch.einsum("hkv,hk->hv", S, k))
                S.add_(k[:, :, None] * u[:, None, :])
                out[t] = torch.einsum("hkv,hk->hv", S, q).reshape(-1)

    def wkv_scan(self, proj, r_off, k_off, v_off, decay, w0, u, state, batch, H, d, out):
        p = proj.float()
        w = torch.exp(-torch.exp(decay[:, :H * d] + w0)).view(-1, H, d)
        uu = u.view(H, d)
        for first, rows, slot, fresh in self._requests(batch):
            if slot < 0:
                out[first:first + rows] = 0
                continue
            S = state[slot, :H * d * d].view(H, d, d)
            if fresh:
                S.zero_()
            for t in range(first, first + rows):
                r = p[t, r_off:r_off + H * d].view(H, d)
                k = p[t, k_off:k_off + H * d].view(H, d)
                v = p[t, v_off:v_off + H * d].view(H, d)
                kv = k[:, :, None] * v[:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S + uu[:, :, None] * kv, r).reshape(-1)
                S.mul_(w[t][:, :, None]).add_(kv)

    def decay_scan(self, proj, q_off, k_off, v_off, decays, state, batch, H, dk, dv, out):
        p = proj.float()
        p = p * torch.sigmoid(p)
        for first, rows, slot, fresh in self._requests(batch):
            if slot < 0:
                out[first:first + rows] = 0
                continue
            S = state[slot, :H * dk * dv].view(H, dk, dv)
            if fresh:
                S.zero_()
            for t in range(first, first + rows):
                q = p[t, q_off:q_off + H * dk].view(H, dk)
                k = p[t, k_off:k_off + H * dk].view(H, dk)
                v = p[t, v_off:v_off + H * dv].view(H, dv)
                S.mul_(decays.float()[:, None, None]).add_(k[:, :, None] * v[:, None, :])
                out[t] = torch.einsum("hkv,hk->hv", S, q).reshape(-1)

    # ---- sublayers that read the stream, results behind a norm
    def stream_cast(self, resid, out):
        out.copy_(resid.to(out.dtype))

    def sum_norm_add(self, xs, scales, weight, eps, resid=None, copy=None):
        y = sum(float(s) * x.float() for x, s in zip(xs, scales))
        if weight is not None:
            y = y * torch.rsqrt((y * y).mean(-1, keepdim=True) + eps) * weight.float()
        if resid is not None:
            resid.add_(y)
            y = resid
        if copy is not None:
            copy.copy_(y.to(copy.dtype))

    def span_rmsnorm(self, x, spans, eps):
        for c0, w, weight, count in spans:
            v = x[:, c0:c0 + w].float()
            v = v * torch.rsqrt((v * v).sum(-1, keepdim=True) / count + eps) * weight.float()
            x[:, c0:c0 + w] = v.to(x.dtype)

    def turn_heads(self, x, heads, head_stride, width, style, positions, inv_freq, sign=1.0, gate=None, gate_stride=0):
        T = x.shape[0]
        v = x[:, :heads * head_stride].float().reshape(T, heads, head_stride).clone()
        if width:
            half = width // 2
            ang = sign * positions.float()[:, None] * inv_freq[:half].float()[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            if style == 0:
                a, b = v[..., :half].clone(), v[..., half:width].clone()
                v[..., :half], v[..., half:width] = a * c - b * s, b * c + a * s
            else:
                a, b = v[..., 0:width:2].clone(), v[..., 1:width:2].clone()
                v[..., 0:width:2], v[..., 1:width:2] = a * c - b * s, b * c + a * s
        if gate is not None:
            g = torch.stack([gate[:, h * gate_stride:h * gate_stride + head_stride].float() for h in range(heads)], dim=1)
            v = v * torch.sigmoid(g)
        x[:, :heads * head_stride] = v.reshape(T, heads * head_stride).to(x.dtype)

    def moe_table_route(self, token_ids, table, ids, weights):
        ids.copy_(table[token_ids.long()])
        weights.fill_(1.0 / ids.shape[1])

    # ---- the token before, gated adds, row norms
    def token_shift(self, h, mu, state, keep_off, batch, out):
        T, width = h.shape
        x = h.float()
        for first, rows, slot, fresh in self._requests(batch):
            kept = state[slot, keep_off:keep_off + width] if slot >= 0 else None
            before = torch.zeros(width) if (kept is None or fresh) else kept.clone()
            prev = torch.cat([before[None, :], x[first:first + rows - 1]], dim=0)
            cur = x[first:first + rows]
            for j in range(mu.shape[0]):
                out[first:first + rows, j * width:(j + 1) * width] = (cur + (prev - cur) * mu[j].float()).to(out.dtype)
            if kept is not None:
                kept.copy_(cur[-1])

    def gated_stream_add(self, resid, gates, a, b=None):
        width = resid.shape[1]
        resid.add_(torch.sigmoid(gates[:, :width].float()) * a.float())
        if b is not None:
            resid.add_(torch.sigmoid(gates[:, width:2 * width].float()) * b.float())

    def rows_rmsnorm(self, x, weight, eps, out):
        v = x.float()
        out.copy_((v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * weight.float()).to(out.dtype))

    def tanh_rows(self, x):
        x.copy_(torch.tanh(x.float()).to(x.dtype))

    def normed_mean(self, outs, weights, eps, out=None, resid=None, scale=1.0):
        y = 0
        for o, w in zip(outs, weights):
            o = o.float()
            y = y + o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * w
        y = y / len(outs)
        if resid is not None:
            resid.add_(scale * y)
        else:
            out.copy_(y.to(out.dtype))

    # ---- mixture of experts
    def moe_route(self, x, router, top, ids, weights, scoring="softmax_chosen", scale=1.0, groups=1, groups_kept=1,
                  group_top=2, correction=None, norm_eps=0.0, outputs=None):
        logits = x.float() @ router.float().T
        z = logits if outputs is None else logits[:, :outputs]
        if scoring == "softmax_chosen":
            val, idx = torch.topk(z, top, dim=-1)
            ids.copy_(idx.to(torch.int32))
            weights.copy_(torch.softmax(val, dim=-1))
            return logits
        if scoring == "softmax":
            s = torch.softmax(z, dim=-1)
            c = s + correction if correction is not None else s.clone()
            T, E = s.shape
            if groups > 1:
                gscore = c.view(T, groups, E // groups).max(-1).values
                kept = torch.topk(gscore, groups_kept, dim=-1).indices
                mask = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, kept, True)
                c = torch.where(mask[:, :, None].expand(T, groups, E // groups).reshape(T, E), c,
                                torch.full_like(c, float("-inf")))
            idx = torch.topk(c, top, dim=-1).indices
            val = torch.gather(s, 1, idx)
            ids.copy_(idx.to(torch.int32))
            weights.copy_(val / (val.sum(-1, keepdim=True) + norm_eps))
            return logits
        s = torch.sigmoid(z)
        T, E = s.shape
        allowed = s
        if groups > 1:
            per = s.view(T, groups, E // groups)
            gscore = torch.topk(per, min(group_top, E // groups), dim=-1).values.sum(-1)
            kept = torch.topk(gscore, groups_kept, dim=-1).indices
            mask = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, kept, True)
            allowed = torch.where(mask[:, :, None].expand(T, groups, E // groups).reshape(T, E), s,
                                  torch.full_like(s, -1.0))
        val, idx = torch.topk(allowed, top, dim=-1)
        ids.copy_(idx.to(torch.int32))
        weights.copy_(val * scale)
        return logits

    def moe_identity_add(self, y, x, ids, weights, experts):
        coef = (weights * (ids >= experts)).sum(-1, keepdim=True)
        y.copy_((y.float() + coef * x.float()).to(y.dtype))

    def moe_silu_gate_scale(self, gu, act, ids, weights, experts, ff, shared, shared_logit=None):
        T = gu.shape[0]
        p = torch.zeros((T, max(experts, int(ids.max()) + 1)))
        p.scatter_(1, ids.long(), weights)
        p = p[:, :experts]
        g = gu[:, :2 * experts * ff].float().view(T, experts, 2, ff)
        a = (g[:, :, 0] * torch.sigmoid(g[:, :, 0]) * g[:, :, 1] * p[:, :, None]).reshape(T, experts * ff)
        if shared:
            sg = gu[:, 2 * experts * ff:].float().view(T, 2, shared)
            sw = torch.sigmoid(shared_logit.float())[:, None] if shared_logit is not None else 1.0
            a = torch.cat([a, sw * sg[:, 0] * torch.sigmoid(sg[:, 0]) * sg[:, 1]], dim=1)
        act.copy_(a.to(act.dtype))

    def moe_relu2_scale(self, up, act, ids, weights, experts, ff):
        T = up.shape[0]
        gate = torch.zeros((T, experts))
        gate.scatter_(1, ids.long(), weights)
        u = torch.relu(up.float()).view(T, experts, ff)
        act.copy_((gate[:, :, None] * u * u).view(T, experts * ff).to(act.dtype))

    def moe_reads_chosen(self, n_tokens, top, experts):
        return n_tokens <= 8 and n_tokens * top <= 0.5 * experts

    def moe_up_chosen(self, x, w_up, ids, weights, act, ff):
        T, top = ids.shape
        for t in range(T):
            for j in range(top):
                e = int(ids[t, j])
                u = torch.relu(w_up[e * ff:(e + 1) * ff].float() @ x[t].float())
                act[t * top + j] = (float(weights[t, j]) * u * u).to(act.dtype)

    def moe_down_chosen(self, act, w_down, ids, ff, resid=None, out=None):
        T, top = ids.shape
        for t in range(T):
            y = sum(w_down[:, int(ids[t, j]) * ff:(int(ids[t, j]) + 1) * ff].float() @ act[t * top + j].float()
                    for j in range(top))
            if resid is not None:
                resid[t] += y
            else:
                out[t] = y.to(out.dtype)

    def moe_gate_up_chosen(self, x, w_gate_up, ids, weights, act, experts, ff, shared, shared_logit=None):
        T, top = ids.shape
        act.zero_()
        for t in range(T):
            xt = x[t].float()
            for j in range(top):
                e = int(ids[t, j])
                if e >= experts:
                    continue
                g = w_gate_up[e * 2 * ff:e * 2 * ff + ff].float() @ xt
                u = w_gate_up[e * 2 * ff + ff:(e + 1) * 2 * ff].float() @ xt
                act[t, j * ff:(j + 1) * ff] = (float(weights[t, j]) * g * torch.sigmoid(g) * u).to(act.dtype)
            if shared:
                b = experts * 2 * ff
                g = w_gate_up[b:b + shared].float() @ xt
                u = w_gate_up[b + shared:].float() @ xt
                sw = torch.sigmoid(shared_logit[t].float()) if shared_logit is not None else 1.0
                act[t, top * ff:] = (sw * g * torch.sigmoid(g) * u).to(act.dtype)

    def moe_down_gated_chosen(self, act, w_down, ids, weights, x, out, experts, ff, shared):
        T, top = ids.shape
        for t in range(T):
            y = torch.zeros(w_down.shape[0])
            for j in range(top):
                e = int(ids[t, j])
                if e >= experts:
                    y += float(weights[t, j]) * x[t].float()
                else:
                    y += w_down[:, e * ff:(e + 1) * ff].float() @ act[t, j * ff:(j + 1) * ff].float()
            if shared:
                y += w_down[:, experts * ff:].float() @ act[t, top * ff:].float()
            out[t] = y.to(out.dtype)

    GATE_GROUP = 8

    def silu_mul(self, gate_up, out, group=0, act="silu", limit=0.0):
        T, I = out.shape
        if group:
            v = gate_up.view(T, I // group, 2, group).float()
            g, u = v[:, :, 0].reshape(T, I), v[:, :, 1].reshape(T, I)
        else:
            g, u = gate_up[:, :I].float(), gate_up[:, I:].float()
        if act == "gelu_tanh":
            a = 0.5 * g * (1 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
        elif act == "swish_bounded":
            g = torch.clamp(g, max=limit)
            a = g * torch.sigmoid(1.702 * g)
            u = torch.clamp(u, min=-limit, max=limit) + 1.0
        else:
            a = g / (1 + torch.exp(-g))
        out.copy_((a * u).to(out.dtype))

    def gated_linear(self, x, weight, out, row_sums=None):
        gu = torch.empty((x.shape[0], weight.shape[0]), dtype=torch.float32)
        self.linear(x, weight, gu)
        if row_sums is not None:
            gu *= self._rstd(row_sums)[:, None]
        self.silu_mul(gu.to(out.dtype), out, self.GATE_GROUP)

    # the accumulating epilogue and the norm that rides on products, so that the parts' use of
    # them runs on the CPU too
    def can_accumulate(self, x, weight):
        return x.shape[0] <= 64

    ROW_PART = 16         # columns of one emitted partial sum
    NORM_ON_PRODUCTS_ROWS = 64

    def skinny_row_parts(self, M, N):
        return -(-N // self._row_part(M))

    def _row_part(self, M):
        return self.ROW_PART if M <= 16 else 1024

    @staticmethod
    def _rstd(row_sums):
        ss, eps, width = row_sums
        return torch.rsqrt(ss.double().sum(0) / width + eps).float()

    def linear_skinny(self, x, weight, out, bias=None, accumulate=False, row_sums=None, emit=None, alpha=1.0):
        y = (x.float() @ weight.float().T) * alpha
        if row_sums is not None:
            y = y * self._rstd(row_sums)[:, None]
        if bias is not None:
            y = y + bias.float()
        if not accumulate:
            assert emit is None
            out.copy_(y.to(out.dtype))
            return
        out.add_(y.to(out.dtype))
        if emit is not None:
            w, xo, so = emit
            xo.copy_((out.float() * w.float()).to(xo.dtype))
            sq = out.float() ** 2
            part = self._row_part(x.shape[0])
            for p in range(so.shape[0]):
                so[p] = sq[:, p * part:(p + 1) * part].sum(1)

    def attention(self, q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads, head_dim,
                  scale, window, group, softcap=0.0, distance=None):
        T = batch.num_tokens
        bs = kcache.shape[2] * 16
        kl, vl = unpack_k(kcache, head_dim), unpack_v(vcache, head_dim)      # [blocks, Hkv, bs, d]
        tables = batch.block_tables[group]
        ratio = num_heads // num_kv_heads
        qh = q[:, :num_heads * head_dim].reshape(T, num_heads, head_dim).float()
        for t in range(T):
            seq = int(batch.seq_of_token[t])
            p = int(batch.positions[t])
            lo = max(0, p - window + 1) if window > 0 else 0
            keys = torch.arange(lo, p + 1)
            blk = tables[seq, keys // bs].long()
            K = kl[blk, :, keys % bs, :].float()        # [n, Hkv, d]
            V = vl[blk, :, keys % bs, :].float()
            for a in range(num_heads):
                s = (K[:, a // ratio, :] @ qh[t, a]) * scale
                if softcap > 0:
                    s = softcap * torch.tanh(s / softcap)
                if distance is not None:
                    s = s - distance[0][a] * torch.log(1.0 + distance[1][a] * (p - keys).float())
                pr = torch.softmax(s, dim=0)
                out[t, a * head_dim:(a + 1) * head_dim] = (pr @ V[:, a // ratio, :]).to(out.dtype)

    attention_plain = attention

    def linear(self, x, weight, out, bias=None):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        out.copy_(y.to(out.dtype))

    linear_plain = linear

    def filter_logits(self, logits, params, histories):
        import plain_qwen3 as plain
        for i, (p, hist) in enumerate(zip(params, histories)):
            win = list(hist[-p.repeat_last_n:]) if p.repeat_last_n > 0 else []
            logits[i] = plain.filter_logits(
                logits[i], max(0.0, p.temperature), top_k=p.top_k or 0, top_p=p.top_p or 0.0,
                min_p=p.min_p or 0.0, repeat_penalty=p.repeat_penalty or 0.0,
                frequency_penalty=p.frequency_penalty or 0.0, presence_penalty=p.presence_penalty or 0.0,
                window=win, logit_bias=p.logit_bias).float()

    def sample(self, logits, temperature, seeds, positions, tokens):
        from plain_qwen3 import mix64, splitmix64, unit_from_u64
        import math
        for r in range(logits.shape[0]):
            T = float(temperature[r])
            best, idx = float("-inf"), -1
            base = splitmix64((int(seeds[r]) & ((1 << 64) - 1)) ^ ((int(positions[r]) * 0x9E3779B97F4A7C15) & ((1 << 64) - 1)))
            for v, x in enumerate(logits[r].tolist()):
                if not math.isfinite(x):
                    continue
                if T > 0:
                    u = unit_from_u64(mix64(base ^ mix64(v)))
                    if u <= 0:
                        continue
                    x = torch.tensor(x, dtype=torch.float32) / torch.tensor(T, dtype=torch.float32) \
                        - torch.log(-torch.log(torch.tensor(u, dtype=torch.float32)))
                    x = float(x)
                if x > best:
                    best, idx = x, v
            tokens[r] = idx
