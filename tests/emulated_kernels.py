"""A stand-in for the device kernels, for tests of the engine's host logic on a
machine without a GPU: the same methods as `llm_rs_amd.kernels.HipKernels`, on CPU
tensors, with the cache layouts and the rounding points of the real kernels.  It
is test equipment: the package never loads it, and the `gpu` tests do not use it.
"""
from __future__ import annotations

import math

import torch

from llm_rs_amd.kernels import Kernels, NormPlan

EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU, EPI_GLU_CLAMP = 0, 1, 2, 3, 5


class EmulatedKernels(Kernels):
    """(What `Kernels` answers by itself stays: no workspace, no scratch, nothing split.)"""

    def embed_rows(self, out, table, tokens, scale=1.0, add=False):
        rows = table[tokens.long()].float() * scale
        out.add_(rows) if add else out.copy_(rows)

    def dyt(self, out, x, weight, bias, alpha, rows=None, second=None):
        src = x if rows is None else x[rows.long()]
        out.copy_((torch.tanh(alpha * src) * weight + bias).to(out.dtype))
        if second is not None:
            out2, w2, b2, a2 = second
            out2.copy_((torch.tanh(a2 * src) * w2 + b2).to(out2.dtype))

    def conv_state_update(self, sums, state, q_starts, slots, channels, taps):
        for e in range(slots.numel()):
            t0, t1 = int(q_starts[e]), int(q_starts[e + 1])
            st = state[int(slots[e])]
            old = st[:(taps - 1) * channels].view(taps - 1, channels)
            old.copy_(torch.cat([old, sums[t0:t1, :channels]])[-(taps - 1):].clone())

    def sigmoid_gate(self, o, gate, per):
        g = torch.sigmoid(gate).repeat_interleave(per, dim=1)
        o.copy_((o.float() * g).to(o.dtype))

    def layernorm(self, out, x, weight, bias, eps, rows=None):
        src = x if rows is None else x[rows.long()]
        dev = src - src.mean(-1, keepdim=True)
        out.copy_((dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * weight + bias).to(out.dtype))

    def latent_finish(self, sums, q, q_size, rank, weight, eps, slot_map, k_cache, v_cache, page_size, num_pages, write,
                      q_weight=None, rotated=None):
        first = sums[:, :q_size]
        if q_weight is not None:
            first = first / torch.sqrt((first * first).mean(-1, keepdim=True) + eps) * q_weight
        q.copy_(first.to(q.dtype))
        if not write:
            return
        c = sums[:, q_size:q_size + rank]
        c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * weight
        if rotated is not None:
            rot, positions, inv_freq, gain = rotated
            part = sums[:, q_size + rank:q_size + rank + rot].clone()
            angle = positions.float()[:, None] * inv_freq[None, :]
            cos, sin = torch.cos(angle) * gain, torch.sin(angle) * gain
            a, b = part[:, 0::2].clone(), part[:, 1::2].clone()
            part[:, 0::2], part[:, 1::2] = a * cos - b * sin, b * cos + a * sin
            c = torch.cat([c, part], dim=1)
        width = c.shape[1]
        kc, vc = k_cache.view(num_pages, page_size, width), v_cache.view(num_pages, width, page_size)
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        for t in range(sums.shape[0]):
            kc[page[t], off[t], :] = c[t].to(kc.dtype)
            vc[page[t], :, off[t]] = c[t].to(vc.dtype)

    def qkv_whole(self, sums, q_cols, k_cols, v_cols, q_weight, k_weight, eps, first=None, lam=None, keep=None):
        for w, lo, n in ((q_weight, 0, q_cols), (k_weight, q_cols, k_cols)):
            if w is not None:
                x = sums[:, lo:lo + n]
                x.copy_(x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w)
        v = sums[:, q_cols + k_cols:q_cols + k_cols + v_cols]
        if first is not None:
            v.copy_((1.0 - lam) * v + lam * first)
        elif keep is not None:
            keep.copy_(v)

    def exp_gates(self, gi, gf, bias_i, bias_f, cap, m_state, q_starts, slots, decay, take, floor):
        i = cap * torch.tanh((gi + (bias_i if bias_i is not None else 0.0)) / cap)
        f = torch.nn.functional.logsigmoid(cap * torch.tanh((gf + (bias_f if bias_f is not None else 0.0)) / cap))
        H = gi.shape[1]
        for e in range(slots.numel()):
            m = m_state[int(slots[e])][:H]
            for t in range(int(q_starts[e]), int(q_starts[e + 1])):
                m_new = torch.maximum(f[t] + m, i[t])
                decay[t], take[t], floor[t] = torch.exp(f[t] + m - m_new), torch.exp(i[t] - m_new), torch.exp(-m_new)
                m.copy_(m_new)

    def head_product(self, a, w, out, gate=None):
        H, n_out, n_in = w.shape
        acc = torch.einsum("thi,hoi->tho", a.float().view(a.shape[0], H, n_in), w.float())
        if gate is not None:
            acc = acc * torch.sigmoid(gate)[:, :, None]
        out.copy_(acc.reshape(a.shape[0], H * n_out).to(out.dtype))

    def scale_softcap_rows(self, logits, scale, cap):
        logits.mul_(scale)
        if cap > 0:
            logits.copy_(cap * torch.tanh(logits / cap))

    def cast(self, dst, src):
        dst.copy_(src.to(dst.dtype))

    def rmsnorm(self, out, x, weight, eps, rows=None):
        src = x if rows is None else x[rows.long()]
        ss = (src * src).sum(-1, keepdim=True)
        inv = 1.0 / torch.sqrt(ss / src.shape[-1] + eps)
        out.copy_((src * inv * weight).to(out.dtype))

    # as the device: steps of up to 16 tokens in bfloat16 leave their norms to the products around them
    def product_norms_its_rows(self, M, N, K, dtype):
        return dtype == torch.bfloat16 and 1 <= M <= 16

    def norm_left_by_product(self, M, N, K, dtype):
        return NormPlan(False, -(-N // 16)) if dtype == torch.bfloat16 and 1 <= M <= 16 else None

    def glu_clamp_slot(self, limit, alpha):
        return (float(limit), float(alpha))          # (no table here: the constants themselves are what gemm is given)

    def gemm(self, a, w, out, epilogue=EPI_STORE, workspace=None, leave=None, glu=None):
        inv = None
        if hasattr(a, "sumsq"):        # kernels.NormedRows: rows times the norm's weight, rounded; the scale comes after the sums
            inv = 1.0 / torch.sqrt(a.sumsq.sum(-1, keepdim=True) / a.y.shape[1] + a.eps)
            a = a.y
        acc = a.float() @ w.float().T
        if inv is not None:
            acc = acc * inv
        if leave is not None:          # kernels.NextNorm, with the += epilogue
            new = out + acc
            pad = torch.zeros((new.shape[0], leave.sumsq.shape[1] * 16))
            pad[:, :new.shape[1]] = new
            leave.sumsq.copy_((pad * pad).view(new.shape[0], -1, 16).sum(-1))
            leave.y.copy_((new * leave.weight).to(leave.y.dtype))
        if epilogue == EPI_STORE:
            out.copy_(acc.to(out.dtype))
        elif epilogue == EPI_STORE_F32:
            out.copy_(acc)
        elif epilogue == EPI_ACCUM_F32:
            out.add_(acc)
        elif epilogue == EPI_GLU_CLAMP:
            limit, alpha = glu
            g, u = torch.clamp(acc[:, 0::2], max=limit), torch.clamp(acc[:, 1::2], min=-limit, max=limit)
            out.copy_((g * torch.sigmoid(alpha * g) * (u + 1.0)).to(out.dtype))
        else:
            g, u = acc[:, 0::2], acc[:, 1::2]
            out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))

    def rope_kv_write(self, qkv, positions, slot_map, inv_freq, rotary_dim, interleaved, k_cache, v_cache,
                      n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv):
        T = qkv.shape[0]
        heads = qkv[:, :(n_heads + 2 * n_kv_heads) * head_dim].view(T, n_heads + 2 * n_kv_heads, head_dim)
        n_rot = n_heads + n_kv_heads
        x = heads[:, :n_rot, :].float()
        if rotary_dim:
            angle = positions.float()[:, None] * inv_freq[None, :]
            cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
            y = x.clone()
            r = rotary_dim
            if interleaved:
                a, b = x[..., 0:r:2], x[..., 1:r:2]
                y[..., 0:r:2], y[..., 1:r:2] = a * cos - b * sin, a * sin + b * cos
            else:
                a, b = x[..., :r // 2], x[..., r // 2:r]
                y[..., :r // 2], y[..., r // 2:r] = a * cos - b * sin, a * sin + b * cos
            x = y
        x = x.to(qkv.dtype)
        heads[:, :n_heads, :] = x[:, :n_heads, :]
        if not write_kv:
            return
        kc = k_cache.view(num_pages, n_kv_heads, page_size, head_dim)
        vc = v_cache.view(num_pages, n_kv_heads, head_dim, page_size)
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        for t in range(T):
            kc[page[t], :, off[t], :] = x[t, n_heads:, :]
            vc[page[t], :, :, off[t]] = heads[t, n_rot:, :]

    def qkv_rope_cache(self, x, w, qkv, positions, slot_map, inv_freq, rotary_dim, k_cache, v_cache,
                       n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv, workspace=None):
        if hasattr(x, "sumsq"):        # the device rotates the 32-bit sums and rounds once; so does this
            full = torch.empty(qkv.shape, dtype=torch.float32)
            self.gemm(x, w, full, EPI_STORE_F32)
            self.rope_kv_write(full, positions, slot_map, inv_freq, rotary_dim, True, k_cache, v_cache,
                               n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv)
            qkv.copy_(full.to(qkv.dtype))
            return
        self.gemm(x, w, qkv, EPI_STORE)
        self.rope_kv_write(qkv, positions, slot_map, inv_freq, rotary_dim, True, k_cache, v_cache,
                           n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv)

    def attention(self, q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens,
                  n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch=None, max_seq_len=0, n_single=-1,
                  single_keys=0, value_dim=0, distance=None, softcap=0.0, keep_first=0, sink=None, gate=None, gate_per=1):
        T = q.shape[0]
        v_dim = value_dim or head_dim
        kc = k_cache.view(num_pages, n_kv_heads, page_size, head_dim).float()
        vc = v_cache.view(num_pages, n_kv_heads, v_dim, page_size).float()
        rep = n_heads // n_kv_heads
        for t in range(T):
            pos = int(positions[t])
            table = block_table[int(token_entry[t])]
            lo = max(0, pos + 1 - window) if window > 0 else 0
            js = torch.cat([torch.arange(0, min(keep_first, lo)), torch.arange(lo, pos + 1)])
            pages, offs = table[js // page_size].long(), js % page_size
            assert int(pages.min()) >= 0, "a visible key's page was given back"
            keys = kc[pages, :, offs, :]                       # [n, kv, d]
            vals = vc[pages, :, :, offs]                       # [n, kv, d]
            qt = q[t, :n_heads * head_dim].view(n_heads, head_dim).float()
            for h in range(n_heads):
                g = h // rep
                s = (keys[:, g, :] @ qt[h]) * scale
                if softcap > 0:
                    s = softcap * torch.tanh(s / softcap)
                if distance is not None:
                    s = s - distance[0][h] * torch.log1p(distance[1][h] * (pos - js).float())
                if sink is not None:         # a key without a value: it only enlarges the denominator
                    p = torch.softmax(torch.cat([s, sink[h:h + 1]]), dim=0)[:-1]
                else:
                    p = torch.softmax(s, dim=0)
                o = p @ vals[:, g, :]
                if gate is not None:         # a number for every gate_per output features: they are multiplied by its sigmoid
                    cols = torch.arange(h * v_dim, (h + 1) * v_dim) // gate_per
                    o = o * (1.0 / (1.0 + torch.exp(-gate[t, cols].float())))
                out[t, h * v_dim:(h + 1) * v_dim] = o.to(out.dtype)

    def group_rmsnorm(self, out, x, weight, eps, groups, rows=None, w_in=None, zero=None, combined=None, mix=None):
        assert x.dim() == 2 and w_in is None and combined is None and mix is None, "one stream only"
        src = x if rows is None else x[rows.long()]
        parts = src.view(src.shape[0], groups, -1)
        inv = 1.0 / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
        out.copy_(((parts * inv).view(src.shape) * weight).to(out.dtype))
        if zero is not None:
            zero.zero_()

    def qkv_finish(self, sums, bias, q, slot_map, k_cache, v_cache, n_heads, n_kv_heads, head_dim, v_dim, page_size, num_pages,
                   write_kv, eps, positions=None, inv_freq=None, rotary_dim=0, q_weight=None, k_weight=None, gain=1.0, conv=None):
        T = sums.shape[0]
        if conv is not None:
            taps, state, q_starts, slots, token_entry = conv
            K, C = taps.shape[1], sums.shape[1]
            x = torch.zeros_like(sums)
            for e in range(slots.numel()):
                t0, t1 = int(q_starts[e]), int(q_starts[e + 1])
                before = state[int(slots[e])][:(K - 1) * C].view(K - 1, C) if K > 1 else sums[:0]
                rows = torch.cat([before, sums[t0:t1]])
                for j in range(K):
                    x[t0:t1] += taps[:, j] * rows[j:j + t1 - t0]
        else:
            x = sums + bias if bias is not None else sums.clone()
        nq, nk = n_heads * head_dim, n_kv_heads * head_dim
        qk = x[:, :nq + nk].reshape(T, n_heads + n_kv_heads, head_dim)
        if eps > 0:
            qk = qk / torch.sqrt((qk * qk).mean(-1, keepdim=True) + eps)
            if q_weight is not None:
                qk[:, :n_heads] = qk[:, :n_heads] * q_weight
            if k_weight is not None:
                qk[:, n_heads:] = qk[:, n_heads:] * k_weight
        if rotary_dim:
            angle = positions.float()[:, None] * inv_freq[None, :]
            cos, sin = torch.cos(angle)[:, None, :] * gain, torch.sin(angle)[:, None, :] * gain
            a, b = qk[..., 0:rotary_dim:2].clone(), qk[..., 1:rotary_dim:2].clone()
            qk[..., 0:rotary_dim:2], qk[..., 1:rotary_dim:2] = a * cos - b * sin, b * cos + a * sin
        q.copy_(qk[:, :n_heads].reshape(T, nq).to(q.dtype))
        if not write_kv:
            return
        kc = k_cache.view(num_pages, n_kv_heads, page_size, head_dim)
        vc = v_cache.view(num_pages, n_kv_heads, v_dim, page_size)
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        vals = x[:, nq + nk:].reshape(T, n_kv_heads, v_dim)
        for t in range(T):
            kc[page[t], :, off[t], :] = qk[t, n_heads:].to(kc.dtype)
            vc[page[t], :, :, off[t]] = vals[t].to(vc.dtype)

    def add_bias_rows(self, rows, bias):
        rows.add_(bias)

    def causal_conv_silu(self, sums, taps, bias, state, q_starts, slots, token_entry, channels, out):
        K = taps.shape[1]
        for e in range(slots.numel()):
            t0, t1 = int(q_starts[e]), int(q_starts[e + 1])
            st = state[int(slots[e])][:(K - 1) * channels].view(K - 1, channels)
            xs = torch.cat([st, sums[t0:t1, :channels]], dim=0)          # the last K - 1 inputs, then this portion's
            for i in range(t1 - t0):
                acc = (taps.T * xs[i:i + K]).sum(0) + (bias if bias is not None else 0.0)
                out[t0 + i] = (acc / (1.0 + torch.exp(-acc))).to(out.dtype)
            if K > 1:
                st.copy_(xs[xs.shape[0] - (K - 1):].clone())

    def silu_columns(self, x, col0, n):
        v = x[:, col0:col0 + n]
        v.copy_(v / (1.0 + torch.exp(-v)))

    def delta_prepare(self, q, k, a, b, A_log, dt_bias, heads, qk_heads, dk, unit_eps):
        T = q.shape[0]
        for x, scale in ((q, dk ** -0.5), (k, 1.0)):
            v = x.reshape(T, qk_heads, dk)
            x.copy_((v / torch.sqrt((v * v).sum(-1, keepdim=True) + unit_eps) * scale).reshape(T, -1))
        z = a.reshape(T, heads, dk) + dt_bias.view(heads, dk)
        soft = torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))
        a.copy_(torch.exp(-torch.exp(A_log)[None, :, None] * soft).reshape(T, -1))
        b.copy_(1.0 / (1.0 + torch.exp(-b)))

    def linear_scan(self, q, k, v, state, q_starts, slots, heads, qk_heads, dk, dv, out, decay=None, g=None, beta=None, gates=None,
                    v_cols=0):
        rep = heads // qk_heads
        if v_cols and v_cols < dv:          # the columns past v's own are written with 1
            v = torch.cat([v.view(-1, heads, v_cols), torch.ones(v.shape[0], heads, dv - v_cols, dtype=v.dtype)], dim=2).reshape(v.shape[0], -1)
        for e in range(slots.numel()):
            S = state[int(slots[e])][:heads * dk * dv].view(heads, dv, dk).transpose(1, 2)       # kept value channel by key channel
            for t in range(int(q_starts[e]), int(q_starts[e + 1])):
                qt = q[t].view(qk_heads, dk).repeat_interleave(rep, dim=0)
                kt = k[t].view(qk_heads, dk).repeat_interleave(rep, dim=0)
                vt = v[t].view(heads, dv)
                if g is not None:
                    S.mul_(g[t].view(heads, dk)[:, :, None])
                elif decay is not None:
                    S.mul_(decay[:, None, None])
                elif gates is not None:
                    S.mul_(gates[0][t][:, None, None])
                    vt = vt * gates[1][t][:, None]
                u = vt if beta is None else beta[t][:, None] * (vt - torch.einsum("hkv,hk->hv", S, kt))
                S.add_(kt[:, :, None] * u[:, None, :])
                out[t] = torch.einsum("hkv,hk->hv", S, qt).reshape(-1)

    def gated_rmsnorm(self, out, x, gate, weight, group, eps, floor=None, x_scale=1.0, den_add=0.0):
        T, W = gate.shape
        if floor is not None:
            wide = x.reshape(T, W // group, group + 1)
            den = torch.maximum(wide[:, :, group].abs() * x_scale, floor) + den_add
            x = (wide[:, :, :group] * x_scale / den[:, :, None]).reshape(T, W)
        parts = x.reshape(T, W // group, group)
        y = (parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)).reshape(T, W)
        w = weight if weight.numel() == W else weight.repeat(W // group)
        out.copy_((y * w / (1.0 + torch.exp(-gate))).to(out.dtype))

    def rmsnorm_sum(self, out, inputs, coef, eps):
        for x, bias, weight in inputs:
            v = x if bias is None else x + bias
            out.add_(coef * v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight)

    def route_topk(self, logits, weights, top, renormalize=False, score="softmax", correction=None, scale=1.0):
        scores = torch.softmax(logits, dim=-1) if score == "softmax" else torch.sigmoid(logits)
        choice = scores if correction is None else scores + correction
        weights.zero_()
        for t in range(logits.shape[0]):
            chosen = sorted(range(logits.shape[1]), key=lambda e: (-float(choice[t, e]), e))[:top]
            total = (sum(float(scores[t, e]) for e in chosen) + (1e-20 if score == "sigmoid" else 0.0)) if renormalize else 1.0
            for e in chosen:
                weights[t, e] = scores[t, e] / total * scale

    def act_weight(self, out, up, weights, ff, activation="relu2", limit=0.0, alpha=1.0):
        if activation == "clamped_glu":
            g, u = torch.clamp(up[:, 0::2], max=limit), torch.clamp(up[:, 1::2], min=-limit, max=limit)
            y = g * torch.sigmoid(alpha * g) * (u + 1.0)
        else:
            y = torch.clamp(up, min=0.0) ** 2
        if weights is not None:
            y = y * weights.repeat_interleave(ff, dim=1)
        out.copy_(y.to(out.dtype))

    def argmax_rows(self, logits, out, scratch=None):
        for i in range(logits.shape[0]):
            best = logits[i].max()
            out[i] = int((logits[i] == best).nonzero()[0])

    def place_ids(self, tokens, rows, sources, ids, vocab):
        for row, src in zip(rows.tolist(), sources.tolist()):
            if 0 <= row < tokens.numel() and 0 <= src < ids.numel() and 0 <= int(ids[src]) < vocab:
                tokens[row] = ids[src]

    def sample_rows(self, logits, words, out):
        w = words.cpu()
        for i in range(logits.shape[0]):
            u = w[i, 0:1].view(torch.float32).item()
            temp = w[i, 1:2].view(torch.float32).item()
            top_k = int(w[i, 2])
            top_p = w[i, 3:4].view(torch.float32).item()
            row = logits[i]
            V = row.shape[0]
            if temp == 0.0:
                out[i] = int((row == row.max()).nonzero()[0])
                continue
            z = row * (1.0 / temp)
            order = sorted(range(V), key=lambda j: (-float(z[j]), j))
            keep = torch.ones(V, dtype=torch.bool)
            if 0 < top_k < V:
                keep[:] = False
                keep[order[:top_k]] = True
            p = torch.softmax(z.masked_fill(~keep, float("-inf")), dim=0)
            if top_p < 1.0:
                total, cut = 0.0, V
                for n, j in enumerate(order):
                    total += float(p[j])
                    if total >= top_p:
                        cut = n + 1
                        break
                p[order[cut:]] = 0.0
                p = p / p.sum()
            hit = (torch.cumsum(p, 0) > u).nonzero()
            out[i] = int(hit[0]) if len(hit) else int(p.nonzero()[-1])
