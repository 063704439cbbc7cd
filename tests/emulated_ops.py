"""Plain torch versions of the kernel table, one function per kernel, written
from each kernel's contract (inputs, layouts, outputs).

Two uses: GPU tests compare each HIP kernel alone with the function of the same
name here; CPU tests plug this table into the engine so that everything above
the kernels (cache manager, block tables, batch packing, step function,
scheduler) runs without a GPU.  Nothing in ``servelab_amd`` imports this file.

Layouts: K pages [pages, nkv, page_size, D]; V pages [pages, nkv, D, page_size];
qkv rows [T, (nh + 2 nkv) D] with q first, then k, then v, head-major.
"""
import numpy as np
import torch


def _f(x):
    return x.float()


class EmulatedOps:
    def __init__(self, act_dtype=torch.float32):
        self.act_dtype = act_dtype

    # ------------------------------------------------------------ embedding
    def embed(self, ids, table, scale=1.0):
        return _f(table[ids.long()]) * scale

    def stream_pair(self, resid, delta, other):
        """[resid + delta | other] as rows in the activation dtype; the streams stay as they are."""
        a = resid if delta is None else resid + _f(delta)
        return torch.cat([a, other], -1).to(self.act_dtype)

    def scale_rows(self, x, factor):
        return x.mul_(factor)

    # ---------------------------------------------------------------- norms
    def add_rmsnorm(self, resid, delta, weight, eps, fuse=False):
        if delta is not None:
            resid += _f(delta)
        var = resid.pow(2).mean(-1, keepdim=True)
        return (resid * torch.rsqrt(var + eps) * weight).to(self.act_dtype)

    def rows_add_rmsnorm(self, resid, delta, rows, weight, eps, fuse=False):
        x = resid[rows.long()]
        if delta is not None:
            x = x + _f(delta[rows.long()])
        var = x.pow(2).mean(-1, keepdim=True)
        return (x * torch.rsqrt(var + eps) * weight).to(self.act_dtype)

    # --------------------------------------------------------------- linear
    def linear(self, x, w, bias, out_f32=False, defer=False):
        y = _f(x) @ _f(w).T
        if bias is not None:
            y = y + bias
        return y if out_f32 else y.to(self.act_dtype)

    def silu_mul(self, gate_up, block=None):
        return self.gate_mul(gate_up, block, "silu")

    @staticmethod
    def _act(z, activation):
        if activation == "silu":
            return z * torch.sigmoid(z)
        if activation == "gelu_tanh":
            return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        return torch.relu(z) if activation == "relu" else torch.relu(z) ** 2

    def gate_mul(self, gate_up, block=None, activation="silu"):
        """gate and up interleaved in blocks of ``block`` columns (default: halves)."""
        T, inter = gate_up.shape[0], gate_up.shape[1] // 2
        block = inter if block is None else block
        gu = _f(gate_up).view(T, inter // block, 2, block)
        g, u = gu[:, :, 0].reshape(T, inter), gu[:, :, 1].reshape(T, inter)
        return (self._act(g, activation) * u).to(self.act_dtype)

    def activate(self, x, activation):
        return x.copy_(self._act(_f(x), activation).to(x.dtype))

    def add_normed_rmsnorm(self, resid, y, y_weight, y_eps, weight, eps, rows=None):
        """v = resid + y / sqrt(mean(y^2) + y_eps) * y_weight; returns v / sqrt(mean(v^2) + eps) *
        weight.  rows None: v goes back into resid; else only those rows, resid untouched."""
        y = _f(y)
        v = resid + y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + y_eps) * y_weight
        if rows is None:
            resid.copy_(v)
        else:
            v = v[rows.long()]
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * weight).to(self.act_dtype)

    def attend_and_project(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                           batch, scale, window, w_out, bias=None, defer=False):
        attn = self.paged_attention(qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                                    batch, scale, window)
        return self.linear(attn, w_out, bias, defer=defer)

    def gated_mlp(self, x, w_gate_up, block, w_down, defer=False, activation="silu", bias_gate_up=None,
                  bias_down=None):
        return self.linear(self.gated_linear(x, w_gate_up, block, activation, bias_gate_up), w_down, bias_down,
                           defer=defer)

    def gated_linear(self, x, w, block, activation="silu", bias=None):
        """(the kernels apply the gate to float32 sums; so does this)"""
        y = _f(x) @ _f(w).T
        if bias is not None:
            y = y + bias
        T, inter = y.shape[0], y.shape[1] // 2
        gu = y.view(T, inter // block, 2, block)
        g, u = gu[:, :, 0].reshape(T, inter), gu[:, :, 1].reshape(T, inter)
        return (self._act(g, activation) * u).to(self.act_dtype)

    # ----------------------------------------------------------------- rope
    def rope_tables(self, positions, inv_freq, magnitude=1.0):
        ang = positions.float()[:, None] * inv_freq[None, :]
        return torch.cos(ang) * magnitude, torch.sin(ang) * magnitude

    def rope_store(self, qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                   pairs8=False, rot_dim=None):
        """Rotate the first ``rot_dim`` channels (default: all) of the q and k
        heads of ``qkv`` in place; write k and v to their pages.  ``pairs8``:
        the rotated channels come in blocks of 8 channels and their 8 partners
        (channel order [block][half][8]) instead of first half, second half."""
        T = qkv.shape[0]
        R = D if rot_dim is None else rot_dim
        half = R // 2
        qk = qkv[:, :(nh + nkv) * D].view(T, nh + nkv, D)
        if cos is not None:
            turned = qk[..., :R]
            if pairs8:
                std = turned.reshape(T, nh + nkv, half // 8, 2, 8).transpose(2, 3).reshape(T, nh + nkv, R)
            else:
                std = turned
            x1, x2 = _f(std[..., :half]), _f(std[..., half:])
            c, s = cos[:, None, :], sin[:, None, :]
            rot = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1).to(qkv.dtype)
            if pairs8:
                rot = rot.reshape(T, nh + nkv, 2, half // 8, 8).transpose(2, 3).reshape(T, nh + nkv, R)
            turned.copy_(rot)
        if k_cache is None:
            return
        k = qkv[:, nh * D:(nh + nkv) * D].view(T, nkv, D)
        v = qkv[:, (nh + nkv) * D:].view(T, nkv, D)
        page, off = (slots // page_size).long(), (slots % page_size).long()
        k_cache[page, :, off, :] = k.to(k_cache.dtype)
        v_cache[page, :, :, off] = v.to(v_cache.dtype)

    def qkv_rope_store(self, x, w, bias, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                       rot_dim=None):
        qkv = self.linear(x, w, bias)
        self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size, True, rot_dim)
        return qkv

    # --------------------------------------------- position encodings of a mixer
    def plan_rotation(self, head_dim, layout):
        """Channels stay as the checkpoint has them, except that an interleaved
        pairing is turned into halves (written independently of the kernel
        table's own: no blocks of 8 here)."""
        import types
        rot = 0 if layout is None else layout.rot_dim
        order = None
        if layout is not None and layout.pairing == "interleaved":
            order = torch.cat([torch.arange(0, rot, 2), torch.arange(1, rot, 2),
                               torch.arange(rot, head_dim)])
        return types.SimpleNamespace(order=order, rot_dim=rot, blocked=False)

    def project_qkv(self, x, w, bias, nh, nkv, D, plan, tables, slots, k_cache, v_cache, page_size,
                    q_scale=1.0):
        assert q_scale == 1.0                # (this table leaves the whole scale to paged_attention)
        qkv = self.linear(x, w, bias)
        cos, sin = (tables.cos, tables.sin) if tables is not None else (None, None)
        self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size, False,
                        plan.rot_dim)
        return qkv

    # ------------------------------------------------------------ attention
    def paged_attention(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                        batch, scale, window):
        T = qkv.shape[0]
        g = nh // nkv
        out = torch.empty(T, nh * D, dtype=self.act_dtype, device=qkv.device)
        cu = batch.cu_q.tolist()
        ctxs = batch.ctx_len.tolist()
        for s in range(batch.num_seqs):
            a, b = cu[s], cu[s + 1]
            ctx = ctxs[s]
            q = _f(qkv[a:b, :nh * D]).view(b - a, nh, D)
            q_pos = batch.positions[a:b].long()
            lo = 0
            if window is not None:
                lo = max(0, int(q_pos[0]) - window + 1)
            k_pos = torch.arange(lo, ctx)
            pages = block_tables[s].long()[k_pos // page_size]
            offs = k_pos % page_size
            k = _f(k_cache[pages, :, offs, :])                     # [ctx', nkv, D]
            v = _f(v_cache[pages, :, :, offs])                     # [ctx', nkv, D]
            k = k.repeat_interleave(g, dim=1)
            v = v.repeat_interleave(g, dim=1)
            scores = torch.einsum("qhd,rhd->hqr", q, k) * scale
            vis = k_pos[None, :] <= q_pos[:, None]
            if window is not None:
                vis &= k_pos[None, :] > q_pos[:, None] - window
            scores = scores.masked_fill(~vis[None], float("-inf"))
            o = torch.einsum("hqr,rhd->qhd", torch.softmax(scores, -1), v)
            out[a:b] = o.reshape(b - a, nh * D).to(self.act_dtype)
        return out

    # ------------------------------------------- deltas, norms on outputs
    def materialize(self, value):
        return value

    def add_into(self, resid, delta):
        resid += _f(delta)

    def add_postnorm(self, resid, y, weight, eps, mult):
        """resid += mult * y / sqrt(mean(y^2) + eps) * weight; returns the stream's rows in the
        activation dtype (y None: only those)."""
        if y is not None:
            y = _f(y)
            resid += mult * (y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps) * weight)
        return resid.to(self.act_dtype)

    def scaled_sum(self, a, sa, b, sb):
        return (sa * _f(a) + sb * _f(b)).to(self.act_dtype)

    def softcap(self, logits, cap):
        return logits.copy_(cap * torch.tanh(logits / cap))

    # --------------------------------------------- matrix memories in state slots
    @staticmethod
    def _sequences(batch):
        """(first row, one past the last row, state slot, whether the sequence starts here)."""
        cu, slots, pos = batch.cu_q.tolist(), batch.state_slots.tolist(), batch.positions.tolist()
        return [(cu[s], cu[s + 1], slots[s], pos[cu[s]] == 0) for s in range(batch.num_seqs)]

    def lowrank_expand(self, buf, col, w2, bias, mode, heads=1, divisor=1.0, rates=None):
        """z = buf[:, col:col + rank] w2^T + bias, float32 [T, C]; "plain": z; "log_sigmoid":
        logsigmoid(z) / divisor; "rate_softplus": -exp(rates[h]) softplus(z), h = c // (C / heads)."""
        C, rank = w2.shape
        z = buf[:, col:col + rank].float() @ w2.T
        if bias is not None:
            z = z + bias
        if mode == "plain":
            return z
        if mode == "log_sigmoid":
            return torch.nn.functional.logsigmoid(z) / divisor
        if mode == "rate_softplus":
            rate = torch.exp(rates).repeat_interleave(C // heads)
            return -rate * torch.nn.functional.softplus(z)
        raise ValueError(mode)

    def short_conv(self, buf, col, taps, state, state_off, batch, write, unit_heads=0, unit_dim=0,
                   unit_eps=1e-6, scaled_heads=0, scale=1.0, bias=None, activation="silu"):
        """silu (``activation`` None: nothing) of a causal convolution over time per channel of buf[:, col:col + C] (taps [C, n],
        the last tap is the token's own); the n - 1 inputs before a step's first token come from
        state[slot, state_off:] laid out [n - 1, C] (oldest first; zeros at a sequence's start) and
        the step's last n - 1 inputs go back there.  The first ``unit_heads`` heads of ``unit_dim``
        channels are then divided by sqrt(sum x^2 + unit_eps); the first ``scaled_heads`` of them
        also multiplied by ``scale``."""
        C, n = taps.shape
        x = buf[:, col:col + C].float()
        out = torch.empty_like(x)
        for a, b, slot, fresh in self._sequences(batch):
            keep = state[slot, state_off:state_off + (n - 1) * C].view(n - 1, C) if n > 1 else torch.zeros(0, C)
            past = torch.zeros(n - 1, C) if fresh else keep.clone()
            full = torch.cat([past, x[a:b]], 0)
            y = sum(full[j:j + b - a] * taps[:, j] for j in range(n))
            if bias is not None:
                y = y + bias
            out[a:b] = y * torch.sigmoid(y) if activation == "silu" else y
            if write and n > 1:
                keep.copy_(full[full.shape[0] - (n - 1):])
        if unit_heads:
            heads = out[:, :unit_heads * unit_dim].view(-1, unit_heads, unit_dim)
            heads /= torch.sqrt(heads.pow(2).sum(-1, keepdim=True) + unit_eps)
            heads[:, :scaled_heads] *= scale
        return out

    def decay_scan(self, src, q_col, k_col, v_col, H, G, D, Dv, log_decay, q_scale, beta_src, beta_col,
                   state, batch, write):
        """Per head S' = diag(exp(log_decay)) S + k v^T and o = S'^T (q_scale q); with
        ``beta_src``: S' = diag(..) S, u = sigmoid(beta) (v - S'^T k), S' += k u^T.  q and k have G
        heads (head h reads h // (H / G)).  The state slot holds S as [H, Dv, D] from 0 on."""
        T = src.shape[0]
        q = src[:, q_col:q_col + G * D].float().view(T, G, D) * q_scale
        k = src[:, k_col:k_col + G * D].float().view(T, G, D)
        v = src[:, v_col:v_col + H * Dv].float().view(T, H, Dv)
        decay = torch.exp(log_decay.view(T, H, D))
        out = torch.empty(T, H, Dv)
        rep = H // G
        for a, b, slot, fresh in self._sequences(batch):
            kept = state[slot, :H * Dv * D].view(H, Dv, D)
            S = torch.zeros(H, Dv, D) if fresh else kept.clone()
            for t in range(a, b):
                kt, qt = k[t].repeat_interleave(rep, 0), q[t].repeat_interleave(rep, 0)
                S = S * decay[t][:, None, :]
                if beta_src is None:
                    u = v[t]
                else:
                    beta = torch.sigmoid(beta_src[t, beta_col:beta_col + H].float())
                    u = beta[:, None] * (v[t] - torch.einsum("hvd,hd->hv", S, kt))
                S = S + u[:, :, None] * kt[:, None, :]
                out[t] = torch.einsum("hvd,hd->hv", S, qt)
            if write:
                kept.copy_(S)
        return out.view(T, H * Dv)

    def mlstm_scan(self, buf, q_col, k_col, v_col, i_col, f_col, H, D, Dv, cap, q_scale, state, batch,
                   write):
        """Matrix memory with exponential gates and a running maximum that starts at 0; the slot
        holds S [H, Dv, D], then n [H, D], then m [H].  Returns S'^T q / (max(|n' . q|, e^-m') + 1e-6)."""
        T = buf.shape[0]
        q = buf[:, q_col:q_col + H * D].float().view(T, H, D) * q_scale
        k = buf[:, k_col:k_col + H * D].float().view(T, H, D)
        v = buf[:, v_col:v_col + H * Dv].float().view(T, H, Dv)
        ig = cap * torch.tanh(buf[:, i_col:i_col + H].float() / cap)
        fg = torch.nn.functional.logsigmoid(cap * torch.tanh(buf[:, f_col:f_col + H].float() / cap))
        out = torch.empty(T, H, Dv)
        nS, nn = H * Dv * D, H * D
        for a, b, slot, fresh in self._sequences(batch):
            row = state[slot]
            if fresh:
                S, n, m = torch.zeros(H, Dv, D), torch.zeros(H, D), torch.zeros(H)
            else:
                S, n, m = row[:nS].view(H, Dv, D).clone(), row[nS:nS + nn].view(H, D).clone(), row[nS + nn:nS + nn + H].clone()
            for t in range(a, b):
                new = torch.maximum(fg[t] + m, ig[t])
                keep, add = torch.exp(fg[t] + m - new), torch.exp(ig[t] - new)
                S = keep[:, None, None] * S + add[:, None, None] * v[t][:, :, None] * k[t][:, None, :]
                n = keep[:, None] * n + add[:, None] * k[t]
                m = new
                den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
                out[t] = torch.einsum("hvd,hd->hv", S, q[t]) / den[:, None]
            if write:
                row[:nS].copy_(S.reshape(-1))
                row[nS:nS + nn].copy_(n.reshape(-1))
                row[nS + nn:nS + nn + H].copy_(m)
        return out.view(T, H * Dv)

    def ssd_scan(self, src, x_col, b_col, c_col, H, G, N, P, steps, step_col, rates, step_bias, skip,
                 state, batch, write):
        """dt = softplus(steps[:, step_col + h] + step_bias[h]); S' = exp(-exp(rates[h]) dt) S +
        dt B x^T; y = S'^T C + skip[h] x.  x [H, P] at x_col of src, B and C [G, N] at b_col and
        c_col (head h reads group h // (H / G)).  The slot holds S as [H, P, N] from 0 on."""
        T = src.shape[0]
        x = src[:, x_col:x_col + H * P].float().view(T, H, P)
        B = src[:, b_col:b_col + G * N].float().view(T, G, N).repeat_interleave(H // G, 1)
        C = src[:, c_col:c_col + G * N].float().view(T, G, N).repeat_interleave(H // G, 1)
        dt = torch.nn.functional.softplus(steps[:, step_col:step_col + H].float() + step_bias)
        keep = torch.exp(-torch.exp(rates) * dt)
        out = torch.empty(T, H, P)
        for a, b, slot, fresh in self._sequences(batch):
            kept = state[slot, :H * P * N].view(H, P, N)
            S = torch.zeros(H, P, N) if fresh else kept.clone()
            for t in range(a, b):
                S = keep[t][:, None, None] * S + (dt[t][:, None] * x[t])[:, :, None] * B[t][:, None, :]
                out[t] = torch.einsum("hpn,hn->hp", S, C[t]) + skip[:, None] * x[t]
            if write:
                kept.copy_(S)
        return out.view(T, H * P)

    def head_norm_gate(self, o, H, Dv, weight, per_head, eps, gate, gate_col, activation, gate_first=False):
        """Each head of o [T, H Dv] (float32) divided by its root mean square, times ``weight``
        ([H Dv] when ``per_head``, else [Dv] for every head), times sigmoid or silu of
        gate[:, gate_col:gate_col + H Dv]."""
        T = o.shape[0]
        x = o.view(T, H, Dv)
        g = gate[:, gate_col:gate_col + H * Dv].float().view(T, H, Dv)
        g = torch.sigmoid(g) if activation == "sigmoid" else g * torch.sigmoid(g)
        if gate_first:              # the gate before the norm
            x = x * g
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        x = x * (weight.view(H, Dv) if per_head else weight)
        if not gate_first:
            x = x * g
        return x.reshape(T, H * Dv).to(self.act_dtype)

    # -------------------------------------- attention with a norm over the projection
    def projnorm_rope_store(self, buf, H, G, D, Dv, q_gain, k_gain, eps, rot, tables, slots, k_cache,
                            v_cache, page_size, values_are_keys=False, conv=None):
        """buf (float32) holds q [H D], k [G D], v [G Dv] side by side.  q and k are RMS-normed over
        all their heads at once, their heads' first ``rot`` channels rotated in halves; k and v go
        to the pages, q is returned [T, H D]."""
        T = buf.shape[0]
        if conv is not None:        # q, k and v first pass a short convolution without an activation
            taps, state, state_off, batch, write = conv
            buf = self.short_conv(buf, 0, taps, state, state_off, batch, write, activation=None)

        def normed(x, gain):
            if gain is None:        # no norm over the projection
                return x
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain

        def turned(x):
            if not rot:
                return x
            half = rot // 2
            c, s = tables.cos[:, None, :], tables.sin[:, None, :]
            a, b = x[..., :half], x[..., half:rot]
            return torch.cat([a * c - b * s, b * c + a * s, x[..., rot:]], -1)
        q = turned(normed(buf[:, :H * D].float(), q_gain).view(T, H, D))
        k = turned(normed(buf[:, H * D:(H + G) * D].float(), k_gain).view(T, G, D))
        v_col = H * D if values_are_keys else (H + G) * D     # (the keys before norm and rotation)
        v = buf[:, v_col:v_col + G * Dv].float().view(T, G, Dv)
        if slots is not None:
            page, off = (slots // page_size).long(), (slots % page_size).long()
            k_cache[page, :, off, :] = k.to(k_cache.dtype)
            v_cache[page, :, :, off] = v.to(v_cache.dtype)
        return q.reshape(T, H * D).to(self.act_dtype)

    def window_attention(self, q, q_col, nh, nkv, Dk, Dv, k_cache, v_cache, page_size, block_tables,
                         batch, scale, window, keep_first=0, slopes=None, sinks=None, gate=None,
                         gate_col=0, softcap=None):
        if slopes is not None or sinks is not None or gate is not None:
            raise NotImplementedError("the emulated window attention has no bias, sink or gate")
        T = q.shape[0]
        g = nh // nkv
        out = torch.empty(T, nh * Dv, dtype=self.act_dtype)
        cu, ctxs = batch.cu_q.tolist(), batch.ctx_len.tolist()
        for s in range(batch.num_seqs):
            a, b = cu[s], cu[s + 1]
            qs = _f(q[a:b, q_col:q_col + nh * Dk]).view(b - a, nh, Dk)
            q_pos = batch.positions[a:b].long()
            k_pos = torch.arange(0, ctxs[s])
            vis = k_pos[None, :] <= q_pos[:, None]
            if window:
                vis &= (k_pos[None, :] > q_pos[:, None] - window) | (k_pos[None, :] < keep_first)
            seen = vis.any(0)
            k_pos, vis = k_pos[seen], vis[:, seen]             # released pages are never read
            pages = block_tables[s].long()[k_pos // page_size]
            offs = k_pos % page_size
            k = _f(k_cache[pages, :, offs, :]).repeat_interleave(g, dim=1)
            if v_cache is None:     # the values are the first Dv channels of the key rows
                v = k[..., :Dv]
            else:
                v = _f(v_cache[pages, :, :, offs]).repeat_interleave(g, dim=1)
            scores = torch.einsum("qhd,rhd->hqr", qs, k) * scale
            if softcap:
                scores = softcap * torch.tanh(scores / softcap)
            scores = scores.masked_fill(~vis[None], float("-inf"))
            o = torch.einsum("hqr,rhd->qhd", torch.softmax(scores, -1), v)
            out[a:b] = o.reshape(b - a, nh * Dv).to(self.act_dtype)
        return out

    # ------------------------------------------------------- a cached latent
    def slice_rmsnorm(self, buf, col, n, gain, eps):
        x = _f(buf[:, col:col + n])
        return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain).to(self.act_dtype)

    def head_products(self, x, x_col, heads, x_head, A, y=None, y_col=0, y_head=None):
        """y[t, h] = A[h] x[t, h]: head h's K values at column x_col + h * x_head of x, its N
        results at column y_col + h * y_head of y."""
        T = x.shape[0]
        H, N, K = A.shape
        y_head = N if y_head is None else y_head
        if y is None:
            y = torch.zeros(T, y_col + heads * y_head, dtype=self.act_dtype)
        for h in range(heads):
            xs = _f(x[:, x_col + h * x_head:x_col + h * x_head + K])
            y[:, y_col + h * y_head:y_col + h * y_head + N] = (xs @ _f(A[h]).T).to(y.dtype)
        return y

    def latent_store(self, buf, nh, D, R, C, down_off, rot, gain, eps, tables, slots, k_cache,
                     page_size, q_out, q_rows=None):
        """The key row of a token: [RMS norm of buf[:, down_off:down_off + C] times gain | the next R
        channels, the first ``rot`` of them turned in halves]; the last R channels of every query
        head (in ``q_rows``, or in buf) turned the same way into q_out[t, h, C:]."""
        T = buf.shape[0]
        q_rows = buf if q_rows is None else q_rows
        half = rot // 2

        def turned(x):              # [..., R]
            if not rot:
                return x
            c, s = tables.cos, tables.sin
            while c.dim() < x.dim():
                c, s = c[:, None], s[:, None]
            a, b = x[..., :half], x[..., half:rot]
            return torch.cat([a * c - b * s, b * c + a * s, x[..., rot:]], -1)
        q = _f(q_rows[:, :nh * (D + R)]).view(T, nh, D + R)
        q_out.view(T, nh, C + R)[:, :, C:] = turned(q[..., D:]).to(q_out.dtype)
        if slots is not None:
            c = _f(buf[:, down_off:down_off + C])
            c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * gain
            row = torch.cat([c, turned(_f(buf[:, down_off + C:down_off + C + R]))], -1)
            page, off = (slots // page_size).long(), (slots % page_size).long()
            k_cache[page, 0, off, :] = row.to(k_cache.dtype)

    # ------------------------------------------------------- routed experts
    def route_tokens(self, logits, experts, top, over_all=False, correction=None, scale=1.0, with_matrices=None):
        """The ``top`` largest of a row's first ``experts`` logits (float32; ties to the lower
        index) and the softmax over them: (chosen [T, top] int32, shares [T, top] float32).
        ``over_all``: the largest softmax shares over all experts plus ``correction``; a chosen one's
        share over the chosen shares' sum (+ 1e-20), times ``scale``."""
        z = logits[:, :experts].float()
        if over_all:
            s = torch.softmax(z, -1)
            pick = torch.topk(s if correction is None else s + correction, top, dim=-1, sorted=True).indices
            w = torch.gather(s, 1, pick)
            return pick.to(torch.int32), w / (w.sum(-1, keepdim=True) + 1e-20) * scale
        best = torch.topk(z, top, dim=-1, sorted=True)
        return best.indices.to(torch.int32), torch.softmax(best.values, -1)

    def routed_experts(self, x, routing, w_gate_up, w_down, base=None, activation="silu", gated=True,
                       base_gate=None, base_gate_col=0, limit=0.0, pass_through=False):
        """sum over a token's choices of share * down_e(act(gate_e x) * up_e x) (+ base);
        w_gate_up [E, 2 ff, width] holds an expert's gate rows before its up rows.  Not gated:
        down_e(act(up_e x)) with w_gate_up [E, ff, width].  base_gate: base times the sigmoid of
        base_gate[t, base_gate_col]."""
        chosen, shares = routing
        T = x.shape[0]
        ff = w_gate_up.shape[1] // 2 if gated else w_gate_up.shape[1]
        xf = _f(x)
        out = torch.zeros(T, w_down.shape[1]) if base is None else _f(base).clone()
        if base_gate is not None:
            out = out * torch.sigmoid(base_gate[:, base_gate_col].float())[:, None]
        for t in range(T):
            for e, s in zip(chosen[t].tolist(), shares[t].tolist()):
                if e >= w_gate_up.shape[0]:         # an expert without matrices hands its input through
                    if not pass_through:
                        raise ValueError("an expert beyond the matrices was chosen")
                    out[t] += s * xf[t]
                    continue
                gu = _f(w_gate_up[e]) @ xf[t]
                if activation == "clamped_swish":
                    g, u = gu[:ff].clamp(max=limit), gu[ff:].clamp(-limit, limit)
                    mid = g * torch.sigmoid(1.702 * g) * (u + 1.0)
                else:
                    mid = self._act(gu[:ff], activation) * gu[ff:] if gated else self._act(gu, activation)
                out[t] += s * (_f(w_down[e]) @ mid.to(self.act_dtype).float())
        return out.to(self.act_dtype)

    # ------------------------------------------------------------- sampling
    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, seeds, draws):
        """One token per row: the argmax where temperature is 0, else the largest
        of ``perturbed_scores`` among the logits the row's cut keeps."""
        out = []
        for r in range(logits.shape[0]):
            T = float(temperature[r])
            if T == 0.0:
                out.append(int(torch.argmax(logits[r])))
                continue
            k = int(top_k[r]) if top_k is not None else -1
            p = float(top_p[r]) if top_p is not None else 1.0
            scores = perturbed_scores(logits[r], T, int(seeds[r]), int(draws[r]))
            scores[~kept_by_cut(logits[r], T, k, p)] = -np.inf
            out.append(int(np.argmax(scores)))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)


def uniform01(seed: int, draw: int, n: int) -> np.ndarray:
    """u_i in (0, 1) for i in [0, n): a counter-based 64-bit mix of (seed, draw, i)
    whose top 23 bits become (bits + 0.5) / 2^23."""
    one = np.ones(n, dtype=np.uint64)
    i = np.arange(n, dtype=np.uint64)
    z = one * np.uint64(seed % (1 << 64)) + np.uint64(0x9E3779B97F4A7C15) * (
        one * np.uint64(draw) * np.uint64(0x100000001B3) + i + np.uint64(1))
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    return ((z >> np.uint64(41)).astype(np.float64) + 0.5) / 8388608.0


def perturbed_scores(row, T: float, seed: int, draw: int) -> np.ndarray:
    """logit_i / max(T, 1e-6) + g_i with g_i = -ln(-ln u_i): the index of the
    largest one is an exact draw from softmax(logits / T) (Gumbel-max)."""
    x = row.detach().double().cpu().numpy() / max(T, 1e-6)
    u = uniform01(seed, draw, x.shape[0])
    return x - np.log(-np.log(u))


def kept_by_cut(row, T: float, top_k: int, top_p: float) -> np.ndarray:
    """Which logits a row's cut keeps: the top_k largest when top_k > 0 (top_p is
    then ignored); else the sorted prefix whose cumulative probability stays
    <= top_p, the first always kept (servelab/engine/sampler.py:30-44)."""
    x = row.detach().double().cpu().numpy() / max(T, 1e-6)
    keep = np.ones(x.shape[0], dtype=bool)
    if top_k > 0:
        keep[:] = False
        keep[np.argsort(-x, kind="stable")[:top_k]] = True
    elif top_p < 1.0:
        order = np.argsort(-x, kind="stable")
        probs = np.exp(x[order] - x[order[0]])
        cum = np.cumsum(probs / probs.sum())
        inside = cum <= top_p
        inside[0] = True
        keep[:] = False
        keep[order[inside]] = True
    return keep
