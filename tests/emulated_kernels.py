"""A stand-in for the HIP library, in torch on the CPU, for tests without a GPU.

It lets the engine's own logic (batch layout, block tables, slot mapping, cache
reuse, scheduling) be tested where no GPU exists. It is not a path of the
product: the engine never selects it; only tests install it with
``ops.set_backend``. Each method does what the kernel of the same name does.
"""
from __future__ import annotations

import math

import torch


class EmulatedBackend:
    name = "emulated"
    device_type = "cpu"

    def embed(self, ids, table, out, scale=1.0):
        rows = table[ids.long()]
        out.copy_(rows if scale == 1.0 else (rows.float() * scale).to(out.dtype))

    def soft_cap(self, x, cap):
        x.copy_(cap * torch.tanh(x / cap))

    def rmsnorm(self, x, residual, residual_mode, w, y, eps):
        s = x.float()
        if residual_mode == 1:
            s = s + residual.float()
        if residual_mode != 0:
            residual.copy_(s.to(residual.dtype))
        r = torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)
        y.copy_(((s * r).to(x.dtype).float() * w.float()).to(x.dtype))

    def silu_mul(self, gu, out):
        I = out.shape[1]
        g, u = gu[:, :I].float(), gu[:, I:].float()
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    def gather_rows(self, x, rows, out):
        out.copy_(x[rows.long()])

    def qk_rope_write(self, qkv, bias, q_norm_w, k_norm_w, eps, cos_sin, rot, positions, slot_mapping,
                      q_out, k_cache, v_cache, Hq, Hkv, D, write_kv, pair_axes=None):
        T = qkv.shape[0]
        dt = qkv.dtype
        x = qkv.float()
        if bias is not None:
            x = (x + bias.float()).to(dt).float()
        q = x[:, :Hq * D].reshape(T, Hq, D)
        k = x[:, Hq * D:(Hq + Hkv) * D].reshape(T, Hkv, D)
        v = x[:, (Hq + Hkv) * D:].reshape(T, Hkv, D)

        def norm(t, w):
            r = torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)
            return ((t * r).to(dt).float() * w.float()).to(dt).float()

        def turn(t):
            if rot == 0:
                return t
            if positions.dim() == 1:
                cs = cos_sin[positions.long()]                # [T, rot]
                cos, sin = cs[:, None, :rot // 2], cs[:, None, rot // 2:]
            else:
                # pair j turns by the coordinate of its axis (axis 0 where no axes are named)
                axes = pair_axes.long() if pair_axes is not None else torch.zeros(rot // 2, dtype=torch.long)
                at = positions.long()[axes].T                 # [T, rot/2]: the position that turns each pair
                j = torch.arange(rot // 2)
                cos, sin = cos_sin[at, j][:, None, :], cos_sin[at, j + rot // 2][:, None, :]
            t1, t2 = t[..., :rot // 2], t[..., rot // 2:rot]
            return torch.cat((t1 * cos - t2 * sin, t2 * cos + t1 * sin, t[..., rot:]), dim=-1)

        if q_norm_w is not None:
            q, k = norm(q, q_norm_w), norm(k, k_norm_w)
        q_out.copy_(turn(q).to(dt))
        if write_kv:
            k = turn(k).to(dt)
            ok = slot_mapping >= 0
            slots = slot_mapping[ok].long()
            k_cache.view(-1, Hkv, D)[slots] = k[ok]
            v_cache.view(-1, Hkv, D)[slots] = v[ok].to(dt)

    def paged_attention(self, q, k_cache, v_cache, out, batch, block_tables, scale, window, chunk=0, cap=0.0, sink=None,
                        gate=None):
        T, Hq, D = q.shape
        page_size, Hkv = k_cache.shape[1], k_cache.shape[2]
        group = Hq // Hkv
        kf = k_cache.reshape(-1, Hkv, D)
        vf = v_cache.reshape(-1, Hkv, v_cache.shape[3])
        for t in range(T):
            r = int(batch.token_req[t])
            p = int(batch.positions[t])
            lo = max(0, p - window + 1) if window > 0 else 0
            if chunk > 0:
                lo = p - p % chunk
            kp = torch.arange(lo, p + 1)
            slots = block_tables[r, kp // page_size].long() * page_size + kp % page_size
            for h in range(Hq):
                kh = kf[slots, h // group].float()
                vh = vf[slots, h // group].float()
                s = (kh @ q[t, h].float()) * scale
                if cap:
                    s = cap * torch.tanh(s / cap)
                if sink is None:
                    o = torch.softmax(s, dim=0) @ vh
                else:
                    m = max(float(s.max()), sink)
                    e = torch.exp(s - m)
                    o = (e @ vh) / (e.sum() + math.exp(sink - m))
                if gate is not None:
                    o = o * torch.sigmoid(gate[0][t, gate[1] + h].float())
                out[t, h] = o.to(out.dtype)

    # -- layers that are not the pre-norm kind
    def scalar_rmsnorm(self, x, gain, y, eps):
        s = x.float()
        y.copy_((s * (gain.float() / torch.sqrt(s.pow(2).mean(-1, keepdim=True) + eps))).to(y.dtype))

    def pair_norm_mean(self, a, wa, b, wb, y, eps):
        def norm(t, w):
            t = t.float()
            return t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w
        y.copy_((0.5 * (norm(a, wa) + norm(b, wb))).to(y.dtype))

    def depth_mix(self, x, a, b, results, index, weights, out, gain, normed, eps, pair=None):
        add = a.float()
        if pair is not None:
            a2, wa, wb, pair_eps = pair
            unit = lambda t: t.float() / torch.sqrt(t.float().pow(2).mean(-1, keepdim=True) + pair_eps)
            add = 0.5 * (unit(a) * wa + unit(a2) * wb)
        if b is not None:
            add = add + b.float()
        if index == 0:
            results[0] = x
        results[index + 1] = x + add
        total = torch.zeros_like(x)
        for j in range(index + 2):
            total = total + weights[j] * results[j]
        out.copy_(total)
        if gain is not None:
            normed.copy_((total * (gain / torch.sqrt(total.pow(2).mean(-1, keepdim=True) + eps))).to(normed.dtype))

    # -- two norms side by side, a hashed pair embedding
    def embed_pair_hash(self, ids, table, pair_table, out, batch, state_slots, prev_state, buckets, mul_prev, mul_cur):
        cu = batch.cu_seqlens_q.tolist()
        for r in range(batch.num_requests):
            lo, hi = cu[r], cu[r + 1]
            if hi <= lo:
                continue
            slot = int(state_slots[r])
            prev = int(prev_state[slot])
            for t in range(lo, hi):
                tok = int(ids[t])
                row = buckets if int(batch.positions[t]) == 0 else (prev * mul_prev + tok * mul_cur) % buckets
                out[t] = table[tok].float() + pair_table[row].float()
                prev = tok
            prev_state[slot] = prev

    def layernorm_pair(self, x, a, b, w1, b1, y1, w2, b2, y2, eps, rows_dtype):
        s = x
        if a is not None:
            s = s + a.float()
        if b is not None:
            s = s + b.float()
        if a is not None or b is not None:
            x.copy_(s)
        mean = s.mean(-1, keepdim=True)
        n = (s - mean) / torch.sqrt(((s - mean) ** 2).mean(-1, keepdim=True) + eps)
        if y1 is not None:
            y1.copy_((n * w1 + b1).to(y1.dtype))
        if y2 is not None:
            y2.copy_((n * w2 + b2).to(y2.dtype))

    def add_streams(self, x, a, b):
        x.add_(a.float() if b is None else a.float() + b.float())

    @staticmethod
    def _act(z, act):
        if act == 1:
            return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        return z * torch.sigmoid(z)

    def act_mul(self, gu, out, act):
        I = out.shape[1]
        out.copy_((self._act(gu[:, :I].float(), act) * gu[:, I:].float()).to(out.dtype))

    # -- attention over a cached latent
    @staticmethod
    def _turn_pairs(t, positions, freqs, gain):
        ang = positions.double()[:, None] * freqs[None, :]
        cos, sin = (ang.cos() * gain).float(), (ang.sin() * gain).float()
        while cos.dim() < t.dim():
            cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
        u, v = t[..., 0::2], t[..., 1::2]
        out = torch.empty_like(t)
        out[..., 0::2] = u * cos - v * sin
        out[..., 1::2] = v * cos + u * sin
        return out

    def latent_prepare(self, a, q_off, q_rank, c_off, kv_rank, rot, wq, wc, eps, freqs, gain, positions, slot_mapping,
                       cache, cq):
        q = a[:, q_off:q_off + q_rank]
        cq.copy_((q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps) * wq).to(cq.dtype))
        if kv_rank == 0 or slot_mapping is None:
            return
        c = a[:, c_off:c_off + kv_rank]
        rows = [c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * wc]
        if rot:
            rows.append(self._turn_pairs(a[:, c_off + kv_rank:c_off + kv_rank + rot], positions, freqs, gain))
        rows = torch.cat(rows, dim=-1).to(cache.dtype)
        ok = slot_mapping >= 0
        cache.view(-1, cache.shape[-1])[slot_mapping[ok].long(), :kv_rank + rot] = rows[ok]

    def head_gemm(self, x, x_off, x_row, w, w_head, w_n, w_k, y, y_off, y_row, gate, gate_off, N, K, turn=None):
        T, H = x.shape[0], x.shape[1]
        m = torch.as_strided(w, (H, N, K), (w_head, w_n, w_k)).float()
        r = torch.einsum("thk,hnk->thn", x[:, :, x_off:x_off + K].float(), m)
        if gate is not None:
            r = r * torch.sigmoid(gate[:, gate_off:gate_off + H])[:, :, None]
        y[:, :, y_off:y_off + N] = r.to(y.dtype)
        return False                               # (the turning is left to rotate_interleaved)

    def rotate_interleaved(self, src, s_off, dst, d_off, rot, freqs, gain, positions):
        dst[:, :, d_off:d_off + rot] = self._turn_pairs(src[:, :, s_off:s_off + rot].float(), positions, freqs, gain).to(dst.dtype)

    # -- a feed-forward of many small experts
    def route_topk(self, logits, ids, scores, bias=None, mode=0):
        if bias is not None:
            logits = logits + bias
        order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :ids.shape[1]]
        ids.copy_(order.to(torch.int32))
        chosen = torch.gather(logits, 1, order)
        scores.copy_(torch.sigmoid(chosen) if mode == 0 else torch.softmax(chosen, dim=-1))

    def experts_gate_up(self, h, ids, scores, gate_up, u, act):
        T, top = ids.shape
        F = gate_up.shape[1] // 2
        for t in range(T):
            for j in range(top):
                e, s = int(ids[t, j]), (scores[t, j] if scores is not None else 1.0)
                gu = gate_up[e].float() @ h[t].float()
                u[t * top + j] = (self._act(s * gu[:F], act) * (s * gu[F:])).to(u.dtype)

    def experts_down(self, u, ids, down, out, weights=None, add=None):
        T, top = ids.shape
        for t in range(T):
            total = torch.zeros(out.shape[1])
            for j in range(top):
                one = down[int(ids[t, j])].float() @ u[t * top + j].float()
                total = total + (one if weights is None else weights[t, j] * one)
            if add is not None:
                total = total + add[t].float()
            out[t] = total.to(out.dtype)

    @staticmethod
    def _turned(t, positions, freqs, sign=1.0):
        half = freqs.shape[0]
        ang = sign * positions.float()[:, None] * freqs[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        u, v = t[..., :half], t[..., half:2 * half]
        return torch.cat((u * cos - v * sin, v * cos + u * sin, t[..., 2 * half:]), dim=-1)

    def rotary_split_write(self, qkv, bias, qk_freqs, rot, v_freqs, positions, slot_mapping, q_out, k_cache, v_cache,
                           Hq, Hkv, D, E, with_kv, more_columns=0, interleaved=False, unit_eps=None, values_from_keys=False,
                           maps=1):
        T, dt = qkv.shape[0], qkv.dtype
        x = qkv.float()
        if more_columns:
            x = x[:, :x.shape[1] - more_columns]
        if bias is not None:
            x = (x + bias.float()).to(dt).float()

        def prepared(t):
            """[T, heads, D] as projected -> turned, made unit vectors"""
            if rot and interleaved:
                ang = positions.float()[:, None] * qk_freqs[None, :]
                cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
                u, w = t[..., 0:rot:2], t[..., 1:rot:2]
                turned = torch.stack((u * cos - w * sin, w * cos + u * sin), dim=-1).flatten(-2)
                t = torch.cat((turned, t[..., rot:]), dim=-1)
            elif rot:
                t = self._turned(t, positions, qk_freqs)
            if unit_eps is not None:
                t = t / torch.sqrt((t * t).mean(-1, keepdim=True) + unit_eps)
            return t

        q = prepared(x[:, :Hq * D].reshape(T, Hq, D))
        if maps > 1:                 # every map a head of its own, with zeros in the other maps' places
            wide = torch.zeros(T, Hq, maps, D)
            for s in range(Hq):
                wide[:, s, s % maps] = q[:, s]
            q = wide.reshape(T, Hq, maps * D)
        q_out.copy_(q.to(dt))
        if with_kv:
            raw_k = x[:, Hq * D:(Hq + Hkv) * D].reshape(T, Hkv, D)
            k = prepared(raw_k).reshape(T, Hkv // maps, maps * D)
            if values_from_keys:
                v = raw_k
            else:
                v = x[:, (Hq + Hkv) * D:].reshape(T, Hkv // maps, E)
            if v_freqs is not None:
                v = self._turned(v, positions, v_freqs)
            ok = slot_mapping >= 0
            slots = slot_mapping[ok].long()
            k_cache.view(-1, Hkv // maps, maps * D)[slots] = k[ok].to(dt)
            v_cache.view(-1, Hkv // maps, E)[slots] = v[ok].to(dt)

    def differential_combine(self, a, lam, out, eps, post, gate=None):
        T, H, E = out.shape
        a = a.float().reshape(T, H, 2, E)
        o = a[:, :, 0] - lam.float() * a[:, :, 1]
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * post
        if gate is not None:
            o = o * torch.sigmoid(gate[0][:, gate[1]:gate[1] + H].float())[:, :, None]
        out.copy_(o.to(out.dtype))

    def gate_rows(self, x, gate):
        x.copy_((x.float() * torch.sigmoid(gate[0][:, gate[1]:gate[1] + x.shape[1]].float())).to(x.dtype))

    def sandwich_step(self, x, y, wb, eps_b, wa, eps_a, h):
        if y is not None:
            yf = y.float()
            x.add_(yf / torch.sqrt((yf * yf).mean(-1, keepdim=True) + eps_b) * wb)
        if wa is not None:
            h.copy_((x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps_a) * wa).to(h.dtype))

    def turn_back(self, x, freqs, positions):
        x.copy_(self._turned(x.float(), positions, freqs, sign=-1.0).to(x.dtype))

    # -- the gated delta rule: the four kernels, request by request and token by token
    def delta_prepare(self, proj, taps, kept, a_lin, dt_bias, a_log, batch, state_slots, q, k, v, beta, H, G, D, E,
                      decay=None, a_col=0):
        n = taps.shape[1]
        Dd = D if decay is None else decay.shape[2]
        into = a_lin if decay is None else decay.view(proj.shape[0], H * Dd)
        C = 2 * G * D + H * E
        x = proj.float()
        for t in range(proj.shape[0]):
            r = int(batch.token_req[t])
            first, pos = int(batch.cu_seqlens_q[r]), int(batch.positions[t])
            mine = kept[int(state_slots[r])]
            total = torch.zeros(C)
            for j in range(n):
                if pos - j < 0:
                    break
                inp = x[t - j, :C] if j <= t - first else mine[:, (n - 1) + (t - first) - j]
                total = total + taps[:, n - 1 - j] * inp
            act = total * torch.sigmoid(total)
            qk = act[:2 * G * D].view(2 * G, D)
            qk = qk / torch.sqrt(qk.pow(2).sum(-1, keepdim=True) + 1e-6)
            q[t] = qk[:G] * D ** -0.5
            k[t] = qk[G:]
            v[t] = act[2 * G * D:].view(H, E)
            step = torch.nn.functional.softplus(a_lin[t, a_col:a_col + H * Dd] + dt_bias, threshold=20.0)
            into[t] = torch.exp(-torch.exp(a_log).repeat_interleave(Dd) * step)
            beta[t] = torch.sigmoid(x[t, C:C + H])

    def conv_state_update(self, proj, kept, n_taps, batch, state_slots, channels):
        x = proj.float()
        for r in range(batch.num_requests):
            first, end = int(batch.cu_seqlens_q[r]), int(batch.cu_seqlens_q[r + 1])
            n = end - first
            if n <= 0 or n_taps == 1:
                continue
            start = int(batch.positions[first])
            mine = kept[int(state_slots[r])]
            old = mine.clone()
            for s in range(n_taps - 1):
                rel = n - (n_taps - 1) + s
                if rel >= 0:
                    mine[:, s] = x[first + rel, :channels]
                else:
                    mine[:, s] = old[:, n + s] if start + rel >= 0 else 0.0

    def delta_rule(self, q, k, v, decay, beta, state, out, batch, state_slots):
        T, G, D = q.shape
        H = v.shape[1]
        for r in range(batch.num_requests):
            first, end = int(batch.cu_seqlens_q[r]), int(batch.cu_seqlens_q[r + 1])
            if end <= first:
                continue
            slot = int(state_slots[r])
            for h in range(H):
                g = h // (H // G)
                S = torch.zeros_like(state[slot, h]) if int(batch.positions[first]) == 0 else state[slot, h].clone()   # [E, D]
                for t in range(first, end):
                    S = S * decay[t, h][None, :]
                    u = beta[t, h] * (v[t, h] - S @ k[t, g])
                    S = S + u[:, None] * k[t, g][None, :]
                    out[t, h] = S @ q[t, g]
                state[slot, h] = S

    def gated_head_norm(self, o, gate, w, y, eps, gate_col=0, gate_act=0):
        T, H, E = o.shape
        z = gate[:, gate_col:gate_col + H * E].reshape(T, H, E)
        r = torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        y.copy_((o * r * w * (z * torch.sigmoid(z) if gate_act == 1 else torch.sigmoid(z))).to(y.dtype))

    # -- several residual streams side by side
    def streams_step(self, X, x0, mix, out_w, a, b, sa, sb, in_w, norm_w, eps, h, total, n, T, W, rows_dtype):
        old = x0[None].expand(n, T, W) if x0 is not None else X
        if mix is not None:
            y = sa * a.float()
            if b is not None:
                y = y + sb * b.float()
            new = torch.einsum("st,srw->trw", mix, old) + out_w[:, None, None] * y[None]
        else:
            new = old.clone()
        if total is not None:
            total.copy_(new.sum(0))
        elif mix is not None or x0 is not None:
            X.copy_(new)
        if h is not None:
            u = new.sum(0) if in_w is None else torch.einsum("s,srw->rw", in_w, new)
            h.copy_((u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * norm_w).to(h.dtype))

    def embed_float(self, ids, table, out, scale):
        out.copy_(table[ids.long()].float() * scale)

    def activation(self, x, act):
        z = x.float()
        if act == 0:
            z = z * torch.sigmoid(z)
        elif act == 1:
            z = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        else:
            z = torch.clamp(z, min=0.0) ** 2
        x.copy_(z.to(x.dtype))

    def scaled_sum(self, a, b, y, sa, sb):
        y.copy_((sa * a.float() + sb * b.float()).to(y.dtype))

    def scale(self, x, factor):
        x.mul_(factor)

    def linear(self, x, w, bias, out):
        y = x.float() @ w.float().T
        if bias is not None:
            y = y + bias.float()
        out.copy_(y.to(out.dtype))

    # products of few rows that take over the residual addition after them and the norm before them
    few_rows = 16
    fuse_norms = True

    def fused_linear(self, x, w, bias, out, gated=False, row_scales=None, residual=None, sum_out=None, ss_out=None, next_w=None):
        dt = x.dtype
        y = x.float() @ w.float().T
        if row_scales is not None:
            ss, eps = row_scales
            y = y * torch.rsqrt(ss.sum(-1, keepdim=True) / x.shape[1] + eps)
        if gated:
            half = w.shape[0] // 2
            g, u = y[:, :half], y[:, half:]
            y = g * torch.sigmoid(g) * u
        elif bias is not None:
            y = y + bias.float()
        if residual is None:
            out.copy_(y.to(out.dtype))
            return
        s = y + residual.float()
        residual.copy_(s.to(residual.dtype))
        sum_out.copy_((s * (next_w.float() if next_w is not None else 1.0)).to(dt))
        pad = (-s.shape[1]) % 16
        ss_out.copy_(torch.nn.functional.pad(s * s, (0, pad)).view(s.shape[0], -1, 16).sum(-1))

    def scale_rows(self, x, squares, eps, out):
        r = torch.rsqrt(squares.sum(-1, keepdim=True) / x.shape[1] + eps)
        out.copy_((x.float() * r).to(out.dtype))

    def sample(self, logits, temperatures, keys, tokens):
        from plain_qwen3 import sample_token
        import math
        mask = (1 << 64) - 1

        def mix(z):
            z = (z + 0x9E3779B97F4A7C15) & mask
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
            return z ^ (z >> 31)

        for r in range(logits.shape[0]):
            temp = float(temperatures[r])
            noise = None
            if temp > 0:
                key = int(keys[r]) & mask
                noise = torch.tensor([-math.log(((mix(key ^ i) >> 40) + 0.5) / 16777216.0)
                                      for i in range(logits.shape[1])], dtype=torch.float32)
            tokens[r] = sample_token(logits[r], temp, noise)
