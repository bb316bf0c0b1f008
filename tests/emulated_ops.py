"""CPU stand-ins for the HIP entry points, with the same signatures and memory layouts.

Used only by tests: they let the host logic of the engine (step building, cache manager,
scheduler, replay) run where there is no GPU, and they are the per-kernel references of
the GPU tests.  Nothing in the package imports this file.
"""
from __future__ import annotations

import torch

MASK64 = (1 << 64) - 1


def _act(g, activation):
    """The activation on the gate branch of a gated product, in its textbook form."""
    if activation == "silu":
        return g / (1.0 + torch.exp(-g))
    if activation == "gelu_tanh":
        return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g)))
    raise ValueError(f"no activation {activation!r}")


class EmulatedOps:

    def __init__(self, dtype=torch.float32, device="cpu"):
        self.dtype = dtype
        self.device = torch.device(device)

    def _r(self, t):  # round to the element type, as a kernel's store does
        return t.to(self.dtype)

    def embed(self, tokens, table, scale=1.0):
        return table[tokens.long()].float() * scale

    SKINNY_ROWS = 64
    DECODE_MAX_GROUP = 16

    def rmsnorm(self, x, weight, eps, rows=None, out_f32=False, partials=None):
        full = x if partials is None else x + partials.sum(0)
        if partials is not None and rows is None:
            x.copy_(full)
        src = full if rows is None else full[rows.long()]
        y = src * (1.0 / torch.sqrt((src * src).sum(-1, keepdim=True) / src.shape[-1] + eps)) * weight
        return y if out_f32 else self._r(y)

    def linear(self, a, w, bias=None, out_f32=False):
        y = a.float() @ w.float().t()
        if bias is not None:
            y = y + bias
        return y if out_f32 else self._r(y)

    def add_partials(self, x, partials):
        x += partials.sum(0)

    def linear_split(self, a, w, allow_partials=True):
        y = a.float() @ w.float().t()
        if a.shape[0] <= self.SKINNY_ROWS and allow_partials:  # two parts, to exercise the consumers
            r = torch.randn(y.shape, generator=torch.Generator().manual_seed(0))
            return torch.stack([y - r, r])
        return y.unsqueeze(0)

    def norm_folds_into(self, M, N, K, n_partials):
        return M <= 16 and N >= 64

    def _normed(self, x, partials, norm_w, eps):
        full = x if partials is None else x + partials.sum(0)
        inv = 1.0 / torch.sqrt((full * full).sum(-1, keepdim=True) / full.shape[-1] + eps)
        return self._r(full * norm_w), inv, (full if partials is not None else None)

    def linear_split_normed(self, x, partials, norm_w, eps, w):
        a, inv, x_new = self._normed(x, partials, norm_w, eps)
        return ((a.float() @ w.float().t()) * inv).unsqueeze(0), x_new

    def linear_swiglu_normed(self, x, partials, norm_w, eps, w_gate_up, intermediate, activation="silu"):
        a, inv, x_new = self._normed(x, partials, norm_w, eps)
        Ip = w_gate_up.shape[0] // 2
        w = w_gate_up.float().view(Ip // 16, 2, 16, -1)
        gate = (a.float() @ w[:, 0].reshape(Ip, -1).t()) * inv
        up = (a.float() @ w[:, 1].reshape(Ip, -1).t()) * inv
        return self._r((_act(gate, activation) * up)[:, :intermediate]), x_new

    def linear_residual(self, a, w, x):
        if a.shape[0] <= self.SKINNY_ROWS:
            return self.linear_split(a, w)
        x += a.float() @ w.float().t()
        return None

    def linear_swiglu(self, a, w_gate_up, intermediate, activation="silu"):
        Ip = w_gate_up.shape[0] // 2
        w = w_gate_up.float().view(Ip // 16, 2, 16, -1)
        gate = a.float() @ w[:, 0].reshape(Ip, -1).t()
        up = a.float() @ w[:, 1].reshape(Ip, -1).t()
        return self._r((_act(gate, activation) * up)[:, :intermediate])

    def rope_kv_write(self, qkv, bias, positions, inv_freq, slot_map, kpool, vpool, H, KV, hd, page_size):
        qkv = qkv if qkv.dim() == 2 else qkv.sum(0)
        if bias is not None:
            qkv = qkv + bias
        T = qkv.shape[0]
        half = hd // 2
        if inv_freq is not None:
            ang = positions.float()[:, None] * inv_freq[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        else:
            c = torch.ones(T, 1, half)
            s = torch.zeros(T, 1, half)

        def rot(x):
            a, b = x[..., :half], x[..., half:]
            return torch.cat([a * c - b * s, a * s + b * c], -1)

        q = self._r(rot(qkv[:, :H * hd].reshape(T, H, hd))).reshape(T, H * hd)
        if slot_map is not None:
            k = self._r(rot(qkv[:, H * hd:(H + KV) * hd].reshape(T, KV, hd)))
            v = self._r(qkv[:, (H + KV) * hd:(H + 2 * KV) * hd].reshape(T, KV, hd))
            page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
            for t in range(T):
                kpool[page[t], :, off[t], :] = k[t]
                vpool[page[t], :, :, off[t]] = v[t]
        return q

    rows_per_block = 64  # flat rows of a work item; a test that hands over a GPU library's work list sets that library's

    def attention_rows_per_block(self, hd):
        return self.rows_per_block

    def layernorm(self, x, weight, bias, eps, rows=None, out_f32=False, partials=None):
        full = x if partials is None else x + partials.sum(0)
        if partials is not None and rows is None:
            x.copy_(full)
        src = full if rows is None else full[rows.long()]
        dev = src - src.mean(-1, keepdim=True)
        y = dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * weight
        if bias is not None:
            y = y + bias
        return y if out_f32 else self._r(y)

    def paged_attention(self, q, kpool, vpool, block_table, seq_q_start, seq_q_len, seq_pos0, work, H, KV, hd,
                        page_size, window, scale, max_key_groups=0, key_splits=0, sinks=None, out_gate=None, chunk=0, softcap=0.0):
        T = q.shape[0]
        g = H // KV
        out = torch.zeros(T, H * hd)
        done = set()
        for s, r0 in work.tolist():
            if s < 0:   # an item that only fills the list up
                continue
            qs, ql, p0 = int(seq_q_start[s]), int(seq_q_len[s]), int(seq_pos0[s])
            for r in range(r0, min(r0 + self.rows_per_block, ql * g)):
                tok, j = divmod(r, g)
                pos = p0 + tok
                lo = 0 if not window else max(0, pos - window + 1)
                if chunk:  # chunks are counted from the request's position 0
                    lo = max(lo, pos // chunk * chunk)
                keys = torch.arange(lo, pos + 1)
                pages = block_table[s].long()[keys // page_size]
                assert (pages >= 0).all(), "attention reads a page that was given back"
                offs = keys % page_size
                for kvh in range(KV):
                    h = kvh * g + j
                    kk = kpool[pages, kvh, offs, :].float()
                    vv = vpool[pages, kvh, :, offs].float()
                    sc = (kk @ q[qs + tok, h * hd:(h + 1) * hd].float()) * scale
                    if softcap:
                        sc = softcap * torch.tanh(sc / softcap)
                    if sinks is not None:  # a term of the denominator without key or value
                        p = torch.softmax(torch.cat([sc, sinks[h].reshape(1).float()]), 0)[:-1]
                    else:
                        p = torch.softmax(sc, 0)
                    o = p @ vv
                    out[qs + tok, h * hd:(h + 1) * hd] = o if out_gate is None else o * out_gate[qs + tok, h]
                    done.add((qs + tok, h))
        assert len(done) == T * H, "the work list does not cover every row and head"
        return self._r(out)

    def decode_attention_fused(self, qkv, bias, inv_freq, slot_map, kpool, vpool, block_table, seq_pos0, H, KV, hd,
                               page_size, window, scale):
        q = self.rope_kv_write(qkv, bias, seq_pos0, inv_freq, slot_map, kpool, vpool, H, KV, hd, page_size)
        return self.decode_attention(q, kpool, vpool, block_table, seq_pos0, H, KV, hd, page_size, window, scale)

    def decode_attention(self, q, kpool, vpool, block_table, seq_pos0, H, KV, hd, page_size, window, scale, sinks=None, out_gate=None,
                         chunk=0, softcap=0.0):
        S = q.shape[0]
        ar = torch.arange(S, dtype=torch.int32)
        work = torch.stack([ar, torch.zeros_like(ar)], 1)
        return self.paged_attention(q, kpool, vpool, block_table, ar, torch.ones_like(ar), seq_pos0, work, H, KV, hd,
                                    page_size, window, scale, sinks=sinks, out_gate=out_gate, chunk=chunk, softcap=softcap)

    # ------------------------------------------------------------------ attention through a latent
    def latent_limits(self):
        return {"row": 15000}

    @staticmethod
    def _rotate_neighbours(x, positions, inv_freq, factor):
        """``x [T, ..., rot]``: pairs (2i, 2i + 1) rotated by ``positions * inv_freq[i]``, cosines and sines times ``factor``."""
        ang = positions.float().reshape([-1] + [1] * (x.dim() - 1)) * inv_freq.float()
        c, sn = torch.cos(ang) * factor, torch.sin(ang) * factor
        u, v = x[..., 0::2], x[..., 1::2]
        return torch.stack([u * c - v * sn, v * c + u * sn], -1).flatten(-2)

    @staticmethod
    def _rotate_halves(x, positions, inv_freq, factor):
        """``x [T, ..., rot]``: pairs (i, i + rot / 2) rotated by ``positions * inv_freq[i]``."""
        ang = positions.float().reshape([-1] + [1] * (x.dim() - 1)) * inv_freq.float()
        c, sn = torch.cos(ang) * factor, torch.sin(ang) * factor
        half = x.shape[-1] // 2
        u, v = x[..., :half], x[..., half:]
        return torch.cat([u * c - v * sn, v * c + u * sn], -1)

    def latent_rows(self, proj, q_norm, c_norm, eps, positions, inv_freq, cs_factor, slot_map, kpool, vpool, q_rank, rank, rot,
                    page_size, halves=False):
        row = proj.sum(0) if proj.dim() == 3 else proj
        T = row.shape[0]
        rms = lambda x: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        cq = torch.zeros(T, -(-q_rank // 8) * 8)
        if q_rank:
            cq[:, :q_rank] = rms(row[:, :q_rank]) * q_norm
        if c_norm is not None:
            c = self._r(rms(row[:, q_rank:q_rank + rank]) * c_norm)
            page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
            kpool[page, 0, off, :rank] = c
            vpool[page, 0, :rank, off] = c
            if rot:
                turn = self._rotate_halves if halves else self._rotate_neighbours
                kpool[page, 0, off, rank:rank + rot] = self._r(turn(row[:, q_rank + rank:q_rank + rank + rot], positions, inv_freq, cs_factor))
        return self._r(cq) if q_rank else None

    def latent_query(self, q, positions, inv_freq, cs_factor, H, d, rot, rank, hd, halves=False):
        T = q.shape[0]
        qh = q.view(T, H, d + rot)
        plain = torch.zeros(T, H, -(-d // 8) * 8)
        plain[..., :d] = qh[..., :d]
        att = torch.full((T, H, hd), float("nan"))  # the first `rank` columns are the per-head product's to fill
        att[..., rank:] = 0.0
        if rot:
            att[..., rank:rank + rot] = (self._rotate_halves if halves else self._rotate_neighbours)(qh[..., d:], positions, inv_freq, cs_factor)
        return self._r(plain), self._r(att)

    def heads_linear(self, a, w, out=None):
        y = torch.einsum("tbk,bnk->tbn", a.float(), w.float())
        if out is None:
            return self._r(y).contiguous()
        out[..., :y.shape[-1]] = self._r(y)
        return out

    # ------------------------------------------------------------------ attention behind a short convolution
    def conv_rows_limits(self):
        return {"row": 15000, "taps": 16}

    def conv_rows(self, proj, conv_w, state, seq_q_start, seq_q_len, seq_slot, positions, unit_norm, eps, temp_coef, temp_every,
                  values_are_keys, gated, slot_map, kpool, vpool, H, KV, d, page_size):
        row = proj.sum(0) if proj.dim() == 3 else proj
        T, C, dp = row.shape[0], (H + KV) * d, kpool.shape[3]
        y = row[:, :C].clone()
        if conv_w is not None:
            taps = conv_w.shape[1]
            for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
                before = state[slot] if taps > 1 else row.new_zeros(0, C)
                hist = torch.cat([before, row[q0:q0 + n, :C]], 0)  # the taps - 1 projected rows before, then the step's
                acc = torch.zeros(n, C)
                for k in range(taps):
                    acc += hist[k:k + n] * conv_w[:, k]
                y[q0:q0 + n] = acc
                if taps > 1:
                    state[slot] = hist[n:]
        q, k = y[:, :H * d].view(T, H, d), y[:, H * d:].view(T, KV, d)
        v = k
        if unit_norm:
            rms = lambda x: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
            q, k = rms(q), rms(k)
        if temp_coef:
            q = q * (1.0 + temp_coef * torch.log(torch.div(positions.long() + 1, temp_every, rounding_mode="floor").float() + 1.0))[:, None, None]
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        for h in range(KV):
            kpool[page, h, off, :d] = self._r(k[:, h])
            if values_are_keys:
                vpool[page, h, :d, off] = self._r(v[:, h])
        qo = torch.zeros(T, H, dp)
        qo[..., :d] = q
        gate = torch.sigmoid(row[:, C:C + H]) if gated else None
        return self._r(qo).view(T, H * dp), gate

    def sample(self, logits, temperature, top_k, top_p, state, any_greedy=True):
        from plain.qwen2_plain import sample as plain_sample
        toks, lps = [], []
        for r in range(logits.shape[0]):
            st = int(state[r].item()) & MASK64
            tok, st = plain_sample(logits[r].numpy(), float(temperature[r]), int(top_k[r]), float(top_p[r]), st)
            state[r] = st - (1 << 64) if st >= (1 << 63) else st
            toks.append(tok)
            lps.append(0.0)
        return torch.tensor(toks, dtype=torch.int32), torch.tensor(lps)

    def top_logprobs(self, logits, inv_t, k):
        lp = torch.log_softmax(logits.double() * inv_t.double()[:, None], -1)
        order = torch.argsort(-logits.double(), dim=-1, stable=True)[:, :k]
        return order.to(torch.int32), torch.gather(lp, 1, order).float()

    def logit_edit(self, logits, row_of, token, delta):
        for r, t, d in zip(row_of.tolist(), token.tolist(), delta.tolist()):
            logits[r, t] += d

    # ------------------------------------------------------------------ a branch's output, normalised, into the stream
    def norm_add(self, x, partials, weight, eps):
        y = partials.sum(0)
        x += y * (1.0 / torch.sqrt((y * y).sum(-1, keepdim=True) / y.shape[-1] + eps)) * weight

    def norm_add_bias(self, x, partials, bias, weight, eps):
        y = partials.sum(0) + (bias if bias is not None else 0.0)
        x += y * (1.0 / torch.sqrt((y * y).sum(-1, keepdim=True) / y.shape[-1] + eps)) * weight

    def pair_norm_add(self, x, pa, wa, pb, wb, weight, eps):
        rms = lambda y: y * (1.0 / torch.sqrt((y * y).sum(-1, keepdim=True) / y.shape[-1] + eps))
        x += rms(0.5 * (rms(pa.sum(0)) * wa + rms(pb.sum(0)) * wb)) * weight

    def gate_mul(self, sums, activation):
        n = sums.shape[1] // 2
        return self._r(_act(sums[:, :n], activation) * sums[:, n:])

    def round_rows(self, x):
        return self._r(x)

    def embed_pair(self, tokens, table, pairs, prev, seq_q_start, seq_q_len, seq_pos0, seq_slot, mul_prev, mul_cur, buckets):
        x = table[tokens.long()].float()
        for q0, n, p0, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_pos0.tolist(), seq_slot.tolist()):
            for j in range(n):
                tok = int(tokens[q0 + j])
                if p0 + j == 0:
                    row = buckets
                else:
                    before = int(tokens[q0 + j - 1]) if j else int(prev[slot])
                    row = (before * mul_prev + tok * mul_cur) % buckets
                x[q0 + j] += pairs[row].float()
            if n:
                prev[slot] = int(tokens[q0 + n - 1])
        return x

    # ------------------------------------------------------------------ q, k and v finished from 32-bit rows
    def finish_rows(self, rows, q_norm, k_norm, eps, positions, inv_freq, rot, neighbours, slot_map, kpool, vpool, H, KV, d, dv, page_size,
                    queries_only=False):
        T, dp = rows.shape[0], kpool.shape[3]
        if queries_only:  # the layer reads another layer's keys and values and writes none
            KV = 0
        nq, nk = H * d, KV * d
        q, k, v = rows[:, :nq], rows[:, nq:nq + nk], rows[:, nq + nk:nq + nk + KV * dv]
        rms = lambda y: y * (1.0 / torch.sqrt((y * y).sum(-1, keepdim=True) / y.shape[-1] + eps))
        if q_norm is not None:
            q = rms(q) * q_norm
        if k_norm is not None:
            k = rms(k) * k_norm
        q, k = q.reshape(T, H, d).clone(), k.reshape(T, KV, d).clone()
        if inv_freq is not None and rot:
            ang = positions.float()[:, None] * inv_freq[None, :]
            c, sn = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            for x in (q, k):
                if neighbours:
                    a, b = x[..., 0:rot:2].clone(), x[..., 1:rot:2].clone()
                    x[..., 0:rot:2], x[..., 1:rot:2] = a * c - b * sn, b * c + a * sn
                else:
                    a, b = x[..., :rot // 2].clone(), x[..., rot // 2:rot].clone()
                    x[..., :rot // 2], x[..., rot // 2:rot] = a * c - b * sn, b * c + a * sn
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        v = v.reshape(T, KV, dv)
        for h in range(KV):
            kpool[page, h, off, :d] = self._r(k[:, h])
            vpool[page, h, :dv, off] = self._r(v[:, h])
        qo = torch.zeros(T, H, dp)
        qo[..., :d] = q
        return self._r(qo).view(T, H * dp)

    # ------------------------------------------------------------------ linear recurrences with gates that depend on the token
    def linrec_limits(self):
        return {"taps": 16, "wkv_dim": 128, "lru_block": 1024}

    def conv_sums(self, sums, col0, channels, bias_in, weight, bias_out, state, seq_q_start, seq_q_len, seq_slot):
        row = (sums.sum(0) if sums.dim() == 3 else sums)[:, col0:col0 + channels]
        if bias_in is not None:
            row = row + bias_in
        taps = weight.shape[1]
        out = torch.zeros(row.shape[0], channels)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            before = state[slot] if taps > 1 else row.new_zeros(0, channels)
            hist = torch.cat([before, row[q0:q0 + n]], 0)
            acc = torch.zeros(n, channels)
            for k in range(taps):
                acc += hist[k:k + n] * weight[:, k]
            out[q0:q0 + n] = acc
            if taps > 1:
                state[slot] = hist[n:]
        return out + bias_out if bias_out is not None else out

    def lru_gates(self, u, wa_t, wi_t, ba, bi, lam, factor):
        T, C = u.shape
        blocks, bw, _ = wa_t.shape
        ub = u.view(T, blocks, bw)
        r = torch.sigmoid(torch.einsum("tbi,bio->tbo", ub, wa_t.float()).reshape(T, C) + ba)
        i = torch.sigmoid(torch.einsum("tbi,bio->tbo", ub, wi_t.float()).reshape(T, C) + bi)
        log_a = -factor * r * torch.nn.functional.softplus(lam)
        return torch.exp(log_a), torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u

    def lru_scan(self, a, drive, y, ycol, y_bias, state, seq_q_start, seq_q_len, seq_slot):
        T, C = a.shape
        out = torch.zeros(T, C)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            S = state[slot].clone()
            for t in range(q0, q0 + n):
                S = a[t] * S + drive[t]
                out[t] = S
            state[slot] = S
        yy = y[:, ycol:ycol + C].float()
        if y_bias is not None:
            yy = yy + y_bias
        return self._r(out * _act(yy, "gelu_tanh"))

    def shift_mix(self, x, prev, mu, seq_q_start, seq_q_len, seq_slot):
        before = torch.zeros_like(x)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            if n:
                before[q0] = prev[slot]
                before[q0 + 1:q0 + n] = x[q0:q0 + n - 1]
                prev[slot] = x[q0 + n - 1]
        return self._r(x[None] + (before - x)[None] * mu[:, None, :])

    def tanh_rows(self, sums):
        return self._r(torch.tanh(sums))

    def wkv(self, r, k, v, gate, z, w0, u, norm_w, eps, state, seq_q_start, seq_q_len, seq_slot, heads, dim):
        T = r.shape[0]
        hv = lambda t: t.float().view(-1, heads, dim)
        r, k, v, g = hv(r), hv(k), hv(v), hv(gate)
        w = torch.exp(-torch.exp(z + w0)).view(T, heads, dim)
        uu = u.view(heads, dim)
        out = torch.zeros(T, heads, dim)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            S = state[slot].clone()
            for t in range(q0, q0 + n):
                kv = k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hi,hij->hj", r[t], S + uu[:, :, None] * kv)
                S = w[t][:, :, None] * S + kv
            state[slot] = S
        o = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps)
        return self._r(o.reshape(T, -1) * norm_w * (g / (1.0 + torch.exp(-g))).reshape(T, -1))

    # ------------------------------------------------------------------ routed experts
    EXPERT_ACTIVATIONS = {"gelu": 0, "gelu_tanh": 1, "silu": 2}

    def route_limits(self):
        return {"experts": 1024, "top": 64}

    def route(self, h, w, bias, top, correction=None, softmax_all=False):
        z = h.float() @ w.t()
        if bias is not None:
            z = z + bias
        if softmax_all:  # scores over every output; a correction for the choice only; the chosen scores over their sum
            score = torch.softmax(z, -1)
            pick = score if correction is None else score + correction
            idx = torch.topk(pick, top, dim=-1).indices
            val = torch.gather(score, 1, idx)
            gates = torch.zeros_like(z)
            gates.scatter_(1, idx, val / (val.sum(-1, keepdim=True) + 1e-20))
            return gates
        val, idx = torch.topk(z, top, dim=-1)
        gates = torch.zeros_like(z)
        gates.scatter_(1, idx, torch.softmax(val, -1))
        return gates

    def expert_act(self, up, gates, ff, activation, experts=None, gated=False):
        T, n = up.shape
        E = gates.shape[1] if experts is None else experts
        mul = None
        if gated:  # the first half of the columns are the gates, the second the up projections
            n //= 2
            up, mul = up[:, :n], up[:, n:]
        if activation == "gelu":
            a = 0.5 * up * (1.0 + torch.erf(up * 0.7071067811865476))
        else:
            a = _act(up, activation)
        if mul is not None:
            a = a * mul
        wgt = torch.ones(T, n)
        wgt[:, :E * ff] = gates[:, :E].repeat_interleave(ff, dim=1)
        return self._r(torch.where(wgt != 0, a * wgt, torch.zeros(())))

    def add_scaled_rows(self, x, h, weights, first, count):
        x += weights[:, first:first + count].sum(-1, keepdim=True) * h.float()

    # ------------------------------------------------------------------ several residual streams
    def streams_read(self, xs, w_in, rows=None):
        src = xs if rows is None else xs[:, rows.long()]
        return src.sum(0) if w_in is None else torch.einsum("s,stw->tw", w_in, src)

    def streams_read_norm(self, xs, w_in, norm_w, eps):
        u = self.streams_read(xs, w_in)
        return self._r(u * (1.0 / torch.sqrt((u * u).sum(-1, keepdim=True) / u.shape[-1] + eps)) * norm_w)

    def streams_write(self, xs, sums, bias, mix, w_out):
        y = sums.sum(0)
        if bias is not None:
            y = y + bias
        xs.copy_(torch.einsum("st,snw->tnw", mix, xs) + w_out[:, None, None] * y[None])

    def streams_write_read_norm(self, xs, sums, bias, mix, w_out, w_in, norm_w, eps):
        self.streams_write(xs, sums, bias, mix, w_out)
        return self.streams_read_norm(xs, w_in, norm_w, eps)

    # ------------------------------------------------------------------ differential attention, state-space duality
    def sigmoid_rows(self, sums):
        return torch.sigmoid(sums)

    def diff_combine(self, o, gate, lam, eps, factor, H, KV, hd, dv, out_cols):
        T, per = o.shape[0], H // KV
        maps = o.float().view(T, KV, 2, per, hd)[..., :dv]  # (key/value head, map, head of the group)
        d = (maps[:, :, 0] - lam * maps[:, :, 1]).reshape(T, H, dv)
        d = d * (1.0 / torch.sqrt((d * d).sum(-1, keepdim=True) / dv + eps)) * factor
        y = torch.zeros(T, out_cols)
        y[:, :H * dv] = d.reshape(T, H * dv) * torch.sigmoid(gate)
        return self._r(y)

    def ssd_limits(self):
        return {"states": 256, "head_dim": 256}

    def ssd_scan(self, xbc, proj, dt_col, dt_bias, a_log, d_skip, state, seq_q_start, seq_q_len, seq_slot, H, P, N, G):
        T = xbc.shape[0]
        act = xbc / (1.0 + torch.exp(-xbc))
        x, B, C = act[:, :H * P].view(T, H, P), act[:, H * P:H * P + G * N].view(T, G, N), act[:, H * P + G * N:].view(T, G, N)
        dt = torch.nn.functional.softplus(proj[:, dt_col:dt_col + H] + dt_bias, threshold=30.0)
        decay = torch.exp(-torch.exp(a_log) * dt)
        group = torch.arange(H) // (H // G)
        y = torch.zeros(T, H, P)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            S = state[slot].clone()
            for t in range(q0, q0 + n):
                S = decay[t][:, None, None] * S + dt[t][:, None, None] * B[t][group][:, :, None] * x[t][:, None, :]
                y[t] = torch.einsum("hnp,hn->hp", S, C[t][group]) + d_skip[:, None] * x[t]
            state[slot] = S
        return y.view(T, H * P)

    def gated_group_norm(self, y, proj, z_col, weight, eps, groups, out_cols):
        T, n = y.shape
        z = proj[:, z_col:z_col + n]
        g = (y * z / (1.0 + torch.exp(-z))).view(T, groups, n // groups)
        g = g * (1.0 / torch.sqrt((g * g).sum(-1, keepdim=True) / (n // groups) + eps))
        out = torch.zeros(T, out_cols)
        out[:, :n] = g.reshape(T, n) * weight
        return self._r(out)

    def softcap(self, logits, scale, cap):
        v = logits * scale
        logits.copy_(cap * torch.tanh(v / cap) if cap > 0 else v)

    # ------------------------------------------------------------------ mixers with state of fixed size
    def recurrent_limits(self):
        return {"taps": 16, "states": 128, "lightning_dim": 256}

    def causal_conv(self, xz, channels, weight, bias, state, seq_q_start, seq_q_len, seq_slot):
        taps = weight.shape[1]
        out = torch.empty(xz.shape[0], channels)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            x = xz[q0:q0 + n, :channels].float()
            hist = torch.cat([state[slot][:taps - 1], x], 0)       # the taps - 1 inputs before, then the step's
            acc = torch.zeros(n, channels) if bias is None else bias.expand(n, channels).clone()
            for k in range(taps):
                acc += hist[k:k + n] * weight[:, k]
            out[q0:q0 + n] = _act(acc, "silu")
            if taps > 1:
                state[slot][:taps - 1] = hist[n:]
        return self._r(out)

    def selective_scan(self, x, xz, dbc, dt_rank, n_states, w_dt, b_dt, a_log, d_skip, state, seq_q_start, seq_q_len, seq_slot):
        T, C = x.shape
        low, B, Cm = dbc[:, :dt_rank], dbc[:, dt_rank:dt_rank + n_states], dbc[:, dt_rank + n_states:]
        dt = torch.nn.functional.softplus(low @ w_dt + (0 if b_dt is None else b_dt))   # w_dt comes transposed, [dt_rank, C]
        A = -torch.exp(a_log)
        xf, z = x.float(), xz[:, C:].float()
        y = torch.empty(T, C)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            S = state[slot].clone()
            for t in range(q0, q0 + n):
                S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * xf[t])[:, None] * B[t][None, :]
                y[t] = S @ Cm[t] + (0 if d_skip is None else d_skip * xf[t])
            state[slot] = S
        return self._r(y * _act(z, "silu"))

    def lightning_attention(self, qkvg, heads, dim, vdim, decay, state, seq_q_start, seq_q_len, seq_slot, chunked=False):
        T = qkvg.shape[0]
        f = qkvg.float()
        q = _act(f[:, :heads * dim], "silu").view(T, heads, dim)
        k = _act(f[:, heads * dim:2 * heads * dim], "silu").view(T, heads, dim)
        v = _act(f[:, 2 * heads * dim:2 * heads * dim + heads * vdim], "silu").view(T, heads, vdim)
        o = torch.empty(T, heads, vdim)
        for q0, n, slot in zip(seq_q_start.tolist(), seq_q_len.tolist(), seq_slot.tolist()):
            S = state[slot].clone()
            for t in range(q0, q0 + n):
                S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
                o[t] = torch.einsum("hde,hd->he", S, q[t])
            state[slot] = S
        return o.reshape(T, heads * vdim)

    def gated_rmsnorm(self, o, gate_of, gate_col, weight, eps):
        n = o.shape[1]
        g = gate_of[:, gate_col:gate_col + n].float()
        return self._r(o * (1.0 / torch.sqrt((o * o).sum(-1, keepdim=True) / n + eps)) * weight * torch.sigmoid(g))

    # ------------------------------------------------------------------ attention whose heads exchange scores
    def talking_limits(self):
        return {"row": 15000}

    def talking_prepare(self, qkv, q_norm, k_norm, eps, positions, inv_freq, rot, cs_factor, v_other, v_lambda, keep_values,
                        slot_map, kpool, vpool, H, KV, d, dv, page_size):
        qkv = qkv if qkv.dim() == 2 else qkv.sum(0)
        T = qkv.shape[0]
        nq, nk, nv = H * d, KV * d, KV * dv
        q, k, v = qkv[:, :nq], qkv[:, nq:nq + nk], qkv[:, nq + nk:nq + nk + nv]
        if q_norm is not None:
            q = q * (1.0 / torch.sqrt((q * q).sum(-1, keepdim=True) / nq + eps)) * q_norm
        if k_norm is not None:
            k = k * (1.0 / torch.sqrt((k * k).sum(-1, keepdim=True) / nk + eps)) * k_norm
        own = v.clone() if keep_values else None
        if v_other is not None:
            v = (1.0 - v_lambda[0]) * v + v_lambda[0] * v_other
        half = rot // 2 if inv_freq is not None else 0

        def rotated(x, heads):
            x = x.reshape(T, heads, d)
            if not half:
                return x
            ang = positions.float()[:, None] * inv_freq[None, :]
            c, s = (torch.cos(ang) * cs_factor)[:, None, :], (torch.sin(ang) * cs_factor)[:, None, :]
            a, b = x[..., :half], x[..., half:2 * half]
            return torch.cat([a * c - b * s, b * c + a * s, x[..., 2 * half:]], -1)

        q = self._r(rotated(q, H)).reshape(T, nq)
        k = self._r(rotated(k, KV))
        v = self._r(v).reshape(T, KV, dv)
        page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
        for t in range(T):
            kpool[page[t], :, off[t], :] = k[t]
            vpool[page[t], :, :, off[t]] = v[t]
        return q, own

    def talking_attention(self, q, kpool, vpool, talk, block_table, seq_q_start, seq_pos0, H, KV, d, dv, page_size, window,
                          keep_first, scale, seq_q_len=None, tiles=False):
        T, S = q.shape[0], seq_q_start.numel()
        rep = H // KV
        out = torch.zeros(T, H, dv)
        starts = seq_q_start.tolist() + [T]
        for s in range(S):
            for t in range(starts[s], starts[s + 1]):
                pos = int(seq_pos0[s]) + t - starts[s]
                lo = max(0, pos - window + 1) if window else 0
                keys = torch.tensor(list(range(min(keep_first, lo))) + list(range(lo, pos + 1)))
                pages = block_table[s].long()[keys // page_size]
                assert (pages >= 0).all(), "attention reads a page that was given back"
                offs = keys % page_size
                kk = kpool[pages, :, offs, :].float()           # [keys, KV, d]
                vv = vpool[pages, :, :, offs].float()           # [keys, KV, dv]
                qq = q[t].float().view(H, d) * scale
                sc = torch.einsum("hd,jhd->hj", qq, kk.repeat_interleave(rep, dim=1))
                if talk is not None:
                    sc = talk @ sc
                p = torch.softmax(sc, -1)
                out[t] = torch.einsum("hj,jhe->he", p, vv.repeat_interleave(rep, dim=1))
        return self._r(out.reshape(T, H * dv))
