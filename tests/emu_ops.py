"""A CPU stand-in for the HIP kernel library, for tests of the engine's logic
(batching, cache pages, block tables, cutting of prompts) on machines without
a GPU.  It follows the kernels' contracts (layouts of the paged cache, what is
float32), not their code, and is installed with ``ops.install_test_double``.
It is not part of the engine and not the plain implementation either.
"""
import torch


class EmuOps:
    def embedding(self, ids, table, scale=1.0):
        return table[ids.long()].float() * scale

    def add_rms_norm(self, resid, delta, weight, eps, out_dtype, rows=None, delta2=None, groups=1, gate=None, base=None, vec=None,
                     weight2=None):
        if gate is not None:
            delta = delta.float() * gate[2] * torch.sigmoid(gate[0].float() + gate[1].float())
        if delta is not None and delta2 is not None:
            delta = delta.float() + delta2.float()
        for more in (base, vec):
            if more is not None:
                more = more.float().expand(resid.shape)
                delta = more if delta is None else delta.float() + more
        if rows is None:
            if delta is not None:
                resid += delta.float()
            x = resid
        else:
            x = resid[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].float()
        xg = x.reshape(x.shape[0], groups, -1)
        r = torch.rsqrt((xg * xg).mean(dim=-1, keepdim=True) + eps)
        normed = (xg * r).reshape(x.shape)
        if weight2 is not None:
            return (normed * weight.float()).to(out_dtype), (normed * weight2.float()).to(out_dtype)
        return (normed * weight.float()).to(out_dtype)

    def scale_cap(self, x, scale=1.0, cap=0.0):
        x.mul_(scale)
        if cap > 0.0:
            x.copy_(cap * torch.tanh(x / cap))
        return x

    def rms_norm(self, x, weight, eps):
        xf = x.float()
        r = torch.rsqrt((xf * xf).mean(dim=-1, keepdim=True) + eps)
        return (xf * r * weight.float()).to(x.dtype)

    def linear(self, x, w, out_dtype=None):
        return (x.float() @ w.float().t()).to(out_dtype or x.dtype)

    def qk_norm_rope_store(self, qkv, n_q, n_kv, d, q_norm_w, k_norm_w, eps, cos, sin, rotary_dim, positions,
                           k_cache, v_cache, page_size, slots):
        T = qkv.shape[0]
        x = qkv.float()
        q = x[:, :n_q * d].reshape(T, n_q, d)
        k = x[:, n_q * d:(n_q + n_kv) * d].reshape(T, n_kv, d)
        v = x[:, (n_q + n_kv) * d:].reshape(T, n_kv, d)
        if q_norm_w is not None:
            q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_norm_w.float()
            k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_norm_w.float()
        if cos is not None:
            half = rotary_dim // 2
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]

            def rot(t):
                a, b, rest = t[..., :half], t[..., half:rotary_dim], t[..., rotary_dim:]
                return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)
            q, k = rot(q), rot(k)
        if slots is not None:
            for t in range(T):
                sl = int(slots[t])
                if sl < 0:
                    continue
                page, off = sl // page_size, sl % page_size
                k_cache[page, :, off, :] = k[t].to(k_cache.dtype)
                v_cache[page, :, :, off] = v[t].to(v_cache.dtype)
        return q.reshape(T, n_q * d).to(qkv.dtype)

    def paged_attention(self, q, k_cache, v_cache, page_size, meta, n_q, n_kv, d, scale, window, softcap=0.0, distance=None,
                        zero_sink=False):
        T = meta.T
        out = torch.zeros((T, n_q, d), dtype=torch.float32)
        qf = q.float().reshape(T, n_q, d)
        bt = meta.block_table
        for t in range(T):
            s = int(meta.token_entry[t])
            p = int(meta.positions[t])
            lo = 0 if not window else max(0, p - window + 1)
            keys = list(range(lo, p + 1))
            pages = [int(bt[s, c // page_size]) for c in keys]
            assert all(pg >= 0 for pg in pages), "attention reads a page that is not held"
            offs = [c % page_size for c in keys]
            K = k_cache[pages, :, offs, :].float()          # [n, n_kv, d]
            V = v_cache[pages, :, :, offs].float()          # [n, n_kv, d]
            for h in range(n_q):
                g = h * n_kv // n_q
                sc = (K[:, g, :] @ qf[t, h]) * scale
                if softcap:
                    sc = softcap * torch.tanh(sc / softcap)
                if distance is not None:
                    back = torch.tensor([p - c for c in keys], dtype=torch.float32)
                    sc = sc - distance[0, h] * torch.log1p(distance[1, h] * back)
                if zero_sink:
                    pr = torch.softmax(torch.cat([sc, torch.zeros(1)]), dim=0)[:-1]
                else:
                    pr = torch.softmax(sc, dim=0)
                out[t, h] = pr @ V[:, g, :]
        return out.reshape(T, n_q * d).to(q.dtype)

    def swiglu(self, gate_up):
        I = gate_up.shape[1] // 2
        g, u = gate_up[:, :I].float(), gate_up[:, I:].float()
        return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)

    def sample(self, logits, temperature, u):
        out = torch.empty(logits.shape[0], dtype=torch.int32)
        for r in range(logits.shape[0]):
            t = float(temperature[r])
            if t == 0.0:
                out[r] = int(torch.argmax(logits[r]))
            else:
                p = torch.softmax(logits[r].double() / t, dim=0)
                c = torch.cumsum(p, 0)
                idx = int(torch.searchsorted(c, torch.tensor(float(u[r]), dtype=torch.float64), right=True))
                out[r] = min(idx, logits.shape[1] - 1)
        return out

    # ---- stream of output-normed layers, kept layer results, recurrences, latent attention ----
    @staticmethod
    def _copy(out, copy_dtype):
        return None if copy_dtype is None or copy_dtype == torch.float32 else out.to(copy_dtype)

    def pair_embedding(self, ids, table, pair, buckets, mul_prev, mul_cur, positions, token_entry, cu_q, slot_ids, last_token,
                       copy_dtype=None):
        out = table[ids.long()].float()
        if pair is not None:
            old = last_token.clone()
            for t in range(ids.shape[0]):
                e = int(token_entry[t])
                if int(positions[t]) == 0:
                    row = buckets
                else:
                    prev = int(old[int(slot_ids[e])]) if t == int(cu_q[e]) else int(ids[t - 1])
                    row = (prev * mul_prev + int(ids[t]) * mul_cur) % buckets
                out[t] += pair[row].float()
            for e in range(slot_ids.shape[0]):
                last_token[int(slot_ids[e])] = ids[int(cu_q[e + 1]) - 1]
        return out, self._copy(out, copy_dtype)

    def norm_residual(self, base, y, weight, eps, out=None, copy_dtype=None, mix=None):
        yf = y.float()
        r = base + yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps) * weight.float()
        if out is None:
            out = r
        else:
            out.copy_(r)
        if mix is not None:
            return self.depth_mix(mix[0], mix[1], mix[2], copy_dtype)
        return out, self._copy(out, copy_dtype)

    def depth_mix(self, kept, n, a, copy_dtype=None):
        out = torch.zeros_like(kept[0])
        for j in range(n):
            out += a[j].float() * kept[j]
        return out, self._copy(out, copy_dtype)

    def xielu(self, x, pq):
        sp = torch.nn.functional.softplus
        z = x.float()
        ap, aq = sp(pq[0].float()), 0.5 + sp(pq[1].float())
        x.copy_(torch.where(z > 0, ap * z * z + 0.5 * z, aq * (torch.expm1(torch.clamp(z, max=0)) - z) + 0.5 * z).to(x.dtype))
        return x

    def mingru(self, zxg, bz, bx, state, pieces, n_pieces, multi, slot_ids):
        W = zxg.shape[1] // 3
        f = zxg.float()
        out = torch.empty((zxg.shape[0], W), dtype=torch.float32)
        pc = pieces.view(4, n_pieces)
        for k in range(n_pieces):
            slot = int(slot_ids[int(pc[0, k])])
            s = state[slot].clone()
            for t in range(int(pc[1, k]), int(pc[2, k])):
                z = torch.sigmoid(f[t, :W] + bz.float())
                u = f[t, W:2 * W] + bx.float()
                c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
                s = (1 - z) * s + z * c
                g = f[t, 2 * W:]
                out[t] = s * g * torch.sigmoid(g)
            state[slot] = s            # pieces come in the order of the tokens, so the state walks through them
        return out.to(zxg.dtype)

    def gemm_strided(self, a, a_strides, b, b_strides, c, c_strides, batch, M, N, K):
        A = torch.as_strided(a, (batch, M, K), a_strides).float()
        B = torch.as_strided(b, (batch, N, K), b_strides).float()
        torch.as_strided(c, (batch, M, N), c_strides).copy_(torch.einsum("bmk,bnk->bmn", A, B).to(c.dtype))
        return c

    @staticmethod
    def _rotate(v, p, freq, mag, dims, interleaved=False):
        if not dims:
            return v
        half = dims // 2
        ang = (p.float()[:, None] * freq[None, :].float())
        c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
        while c.dim() < v.dim():
            c, s = c[:, None], s[:, None]
        if interleaved:
            a, b = v[..., 0:dims:2], v[..., 1:dims:2]
            turned = torch.stack([a * c - b * s, b * c + a * s], dim=-1).flatten(-2)
            return torch.cat([turned, v[..., dims:]], dim=-1)
        a, b = v[..., :half], v[..., half:dims]
        return torch.cat([a * c - b * s, b * c + a * s, v[..., dims:]], dim=-1)

    def latent_prepare(self, q, dkv, cache, slot_mapping, w_norm, eps, freq, mag, dims, positions, H, DN, DR, R, qa_dtype=torch.float32,
                       interleaved=False):
        T = q.shape[0]
        qa = torch.zeros((T, H, R + DR), dtype=torch.float32)
        qh = q[:, :H * (DN + DR)].float().reshape(T, H, DN + DR)
        qa[:, :, R:] = self._rotate(qh[:, :, DN:], positions, freq, mag, dims, interleaved)
        if dkv is not None:
            d = dkv.float()
            c = d[:, :R] * torch.rsqrt((d[:, :R] ** 2).mean(-1, keepdim=True) + eps) * w_norm.float()
            rows = torch.cat([c, self._rotate(d[:, R:], positions, freq, mag, dims, interleaved)], dim=-1).to(cache.dtype)
            P = cache.shape[1]
            for t in range(T):
                sl = int(slot_mapping[t])
                cache[sl // P, sl % P] = rows[t]
        return qa

    def latent_attention(self, qa, cache, page_size, meta, sink, R, scale, window, out_dtype):
        T, H, D = qa.shape
        out = torch.zeros((T, H, R), dtype=torch.float32)
        for t in range(T):
            s, p = int(meta.token_entry[t]), int(meta.positions[t])
            lo = 0 if not window else max(0, p - window + 1)
            keys = list(range(lo, p + 1))
            pages = [int(meta.block_table[s, c // page_size]) for c in keys]
            assert all(pg >= 0 for pg in pages), "attention reads a page that is not held"
            rows = cache[pages, [c % page_size for c in keys]].float()
            sc = (qa[t] @ rows.T) * scale                                  # [H, n]
            if sink is not None:
                sc = torch.cat([sc, sink.float()[:, None]], dim=1)
            pr = torch.softmax(sc, dim=1)[:, :len(keys)]
            out[t] = pr @ rows[:, :R]
        return out.to(out_dtype)

    # ---- attention with biases, angles formed per call, an output gate ----
    def bias_rope_store(self, x, n_q, n_kv, d, bias, freq, rotary_dim, positions, k_cache, v_cache, page_size, slots, mag=1.0,
                        value_norm=None, query_temperature=None):
        T = x.shape[0]
        n = (n_q + 2 * n_kv) * d
        f = x[:, :n].float()
        if bias is not None:
            f = f + bias.float()
        q = f[:, :n_q * d].reshape(T, n_q, d)
        k = f[:, n_q * d:(n_q + n_kv) * d].reshape(T, n_kv, d)
        v = f[:, (n_q + n_kv) * d:].reshape(T, n_kv, d)
        if rotary_dim:
            q, k = self._rotate(q, positions, freq, mag, rotary_dim), self._rotate(k, positions, freq, mag, rotary_dim)
        if value_norm is not None:
            eps, n = value_norm
            v = v * torch.rsqrt((v[..., :n] ** 2).mean(-1, keepdim=True) + eps)
        if query_temperature is not None:
            coef, every = query_temperature
            steps = torch.div(positions.long() + 1, int(every), rounding_mode="floor").float()
            q = q * (1.0 + coef * torch.log(steps + 1.0))[:, None, None]
        if slots is not None:
            for t in range(T):
                sl = int(slots[t])
                if sl < 0:
                    continue
                k_cache[sl // page_size, :, sl % page_size, :] = k[t].to(k_cache.dtype)
                v_cache[sl // page_size, :, :, sl % page_size] = v[t].to(v_cache.dtype)
        return q.reshape(T, n_q * d).to(x.dtype)

    def sigmoid_gate(self, y, gate, bias=None, mult=1.0, per=1):
        g = gate.float() if bias is None else gate.float() + bias.float()
        g = g.repeat_interleave(per, dim=1) if per > 1 else g
        y.copy_((y.float() * torch.sigmoid(g) * mult).to(y.dtype))
        return y

    # ---- matrix memories ----
    def mlstm(self, x, q_off, k_off, v_off, g_off, gates, bi, bf, cap, norm_w, eps, state, cu_q, slot_ids, H, d, dv, pieces=None):
        T = x.shape[0]
        f = x.float()
        out = torch.zeros((T, H, dv), dtype=torch.float32)
        for s in range(slot_ids.shape[0]):
            st = state[int(slot_ids[s])].view(H, -1)          # per head: S, then (n, m) once per slice of value channels
            for h in range(H):
                S, n, m = st[h, :d * dv].view(d, dv).clone(), st[h, d * dv:d * dv + d].clone(), float(st[h, d * dv + d])
                for t in range(int(cu_q[s]), int(cu_q[s + 1])):
                    q = f[t, q_off + h * d:q_off + (h + 1) * d] * d ** -0.5
                    k = f[t, k_off + h * d:k_off + (h + 1) * d]
                    v = f[t, v_off + h * dv:v_off + (h + 1) * dv]
                    ig = cap * torch.tanh((gates[t, h] + bi[h].float()) / cap)
                    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((gates[t, H + h] + bf[h].float()) / cap))
                    m_new = max(float(fg) + m, float(ig))
                    a, b = torch.exp(fg + m - m_new), torch.exp(ig - m_new)
                    S = a * S + b * torch.outer(k, v)
                    n = a * n + b * k
                    m = m_new
                    den = max(abs(float(n @ q)), float(torch.exp(torch.tensor(-m)))) + 1e-6
                    out[t, h] = (S.T @ q) / den
                st[h, :d * dv] = S.reshape(-1)
                for c in range((st.shape[1] - d * dv) // (d + 1)):
                    st[h, d * dv + c * (d + 1):d * dv + c * (d + 1) + d] = n
                    st[h, d * dv + c * (d + 1) + d] = m
        out = out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps)
        g = f[:, g_off:g_off + H * dv]
        return (out.reshape(T, H * dv) * norm_w.float() * torch.sigmoid(g)).to(x.dtype)

    def causal_conv_silu(self, x, taps, state, keep_off, token_entry, cu_q, slot_ids):
        T, C = x.shape
        n = taps.shape[1]
        f = x.float()
        y = torch.zeros((T, C), dtype=torch.float32)
        for s in range(slot_ids.shape[0]):
            keep = state[int(slot_ids[s]), keep_off:keep_off + (n - 1) * C].view(n - 1, C)
            t0, t1 = int(cu_q[s]), int(cu_q[s + 1])
            rows = torch.cat([keep.clone(), f[t0:t1]], dim=0)
            for t in range(t1 - t0):
                acc = (rows[t:t + n] * taps.float().T).sum(0)
                y[t0 + t] = acc * torch.sigmoid(acc)
            if n > 1:
                keep.copy_(rows[rows.shape[0] - (n - 1):])
        return y.to(x.dtype)

    def delta_rule(self, qkv, beta_pre, dec_pre, a_log, dt_bias, gate, norm_w, eps, state, cu_q, slot_ids, H, G, d, dv, gate_act="sigmoid"):
        T = qkv.shape[0]
        f = qkv.float()
        q = f[:, :G * d].reshape(T, G, d)
        k = f[:, G * d:2 * G * d].reshape(T, G, d)
        v = f[:, 2 * G * d:].reshape(T, H, dv)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(beta_pre)
        dec = torch.exp(-torch.exp(a_log.float())[None, :, None] * torch.nn.functional.softplus(dec_pre + dt_bias.float()).view(T, H, -1))
        dec = dec.expand(T, H, d)              # (one decay per head: the same for all its key channels)
        out = torch.zeros((T, H, dv), dtype=torch.float32)
        for s in range(slot_ids.shape[0]):
            st = state[int(slot_ids[s]), :H * d * dv].view(H, d, dv)
            for h in range(H):
                g = h // (H // G)
                S = st[h].clone()
                for t in range(int(cu_q[s]), int(cu_q[s + 1])):
                    S = dec[t, h][:, None] * S
                    u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
                    S = S + torch.outer(k[t, g], u)
                    out[t, h] = S.T @ q[t, g]
                st[h] = S
        out = out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps) * norm_w.float()
        g = gate.float()
        return (out.reshape(T, H * dv) * (torch.sigmoid(g) if gate_act == "sigmoid" else g * torch.sigmoid(g))).to(qkv.dtype)

    # ---- token shift and the state with a decay per key channel ----
    def token_shift(self, x, mu, state, keep_off, token_entry, cu_q, slot_ids):
        T, W = x.shape
        f = x.float()
        prev = torch.zeros_like(f)
        for s in range(slot_ids.shape[0]):
            keep = state[int(slot_ids[s]), keep_off:keep_off + W]
            t0, t1 = int(cu_q[s]), int(cu_q[s + 1])
            prev[t0] = keep
            prev[t0 + 1:t1] = f[t0:t1 - 1]
            keep.copy_(f[t1 - 1])
        return (f[None] + (prev - f)[None] * mu.float()[:, None, :]).to(x.dtype)

    def tanh_cast(self, x, dtype):
        return torch.tanh(x).to(dtype)

    def time_mix(self, r, k, v, dec_pre, w0, u, gate, norm_w, eps, state, cu_q, slot_ids, H, d):
        T = r.shape[0]
        rf, kf, vf = (t.float().reshape(T, H, d) for t in (r, k, v))
        dec = torch.exp(-torch.exp(dec_pre + w0.float())).view(T, H, d)
        uu = u.float().view(H, d)
        out = torch.zeros((T, H, d), dtype=torch.float32)
        for s in range(slot_ids.shape[0]):
            st = state[int(slot_ids[s]), :H * d * d].view(H, d, d)
            S = st.clone()
            for t in range(int(cu_q[s]), int(cu_q[s + 1])):
                kv = kf[t][:, :, None] * vf[t][:, None, :]
                out[t] = torch.einsum("hi,hij->hj", rf[t], S + uu[:, :, None] * kv)
                S = dec[t][:, :, None] * S + kv
            st.copy_(S)
        out = out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps)
        g = gate.float()
        return (out.reshape(T, H * d) * norm_w.float() * g * torch.sigmoid(g)).to(r.dtype)

    def norm_pair_mean(self, a, b, wa, wb, eps):
        af, bf = a.float(), b.float()
        na = af * torch.rsqrt((af * af).mean(-1, keepdim=True) + eps) * wa.float()
        nb = bf * torch.rsqrt((bf * bf).mean(-1, keepdim=True) + eps) * wb.float()
        return (0.5 * (na + nb)).to(a.dtype)

    # ---- mixture of experts ----
    def moe_route(self, z, correction, top, groups, keep, scale, score="softmax", renormalize=True, logit_bias=None):
        T, E = z.shape
        if logit_bias is not None:
            z = z.float() + logit_bias.float()
        per = E // groups
        ids = torch.zeros((T, top), dtype=torch.int32)
        w = torch.zeros((T, top), dtype=torch.float32)
        for t in range(T):
            s = torch.softmax(z[t].float(), dim=0) if score == "softmax" else torch.sigmoid(z[t].float())
            ch = (s + correction.float()).tolist() if correction is not None else s.tolist()
            best = sorted(range(groups), key=lambda g: (-max(ch[g * per:(g + 1) * per]), g))[:keep]
            allowed = [e for e in range(E) if e // per in best]
            chosen = sorted(allowed, key=lambda e: (-ch[e], e))[:top]
            tot = (sum(float(s[e]) for e in chosen) + 1e-20) if renormalize else 1.0
            for j, e in enumerate(chosen):
                ids[t, j], w[t, j] = e, float(s[e]) / tot * scale
        return ids, w

    def moe_experts(self, x, ids, weights, w_gate_up, w_down, activation="silu", limit=0.0, weight_input=False, add=None):
        T, K = x.shape
        F = w_gate_up.shape[1] // 2
        out = torch.zeros((T, K), dtype=torch.float32)
        xf = x.float()
        for t in range(T):
            for j in range(ids.shape[1]):
                e = int(ids[t, j])
                gu = w_gate_up[e].float() @ xf[t]
                if weight_input:
                    gu = gu * weights[t, j]
                if activation == "silu":
                    act = gu[:F] * torch.sigmoid(gu[:F]) * gu[F:]
                else:
                    g, u = torch.clamp(gu[:F], max=limit), torch.clamp(gu[F:], -limit, limit)
                    act = g * torch.sigmoid(1.702 * g) * (u + 1.0)
                act = act.to(x.dtype).float()
                out[t] += (1.0 if weight_input else weights[t, j]) * (w_down[e].float() @ act)
        if add is not None:
            out += add.float()
        return out.to(x.dtype)
