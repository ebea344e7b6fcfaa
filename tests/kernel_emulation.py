"""A test double for the kernel library: the same calls, computed with torch on the CPU.

It exists so that the engine's own logic (step layout, paged cache, slots, generation loop)
can be tested where there is no GPU.  It is slow and lives under tests/: the product has no
CPU path, and nothing in the package imports this file.
"""

from __future__ import annotations

import torch

PAGE = 64


class TorchKernels:
    page_size = PAGE

    def __init__(self, device="cpu"):
        self.device = torch.device(device)
        self.calls = []

    def embed(self, tokens, table, out):
        self.calls.append("embed")
        out.copy_(table[tokens.long()].float())

    def rmsnorm(self, x, weight, eps, out, rows=None):
        self.calls.append("rmsnorm")
        src = x if rows is None else x[rows.long()]
        inv = 1.0 / torch.sqrt((src.double() ** 2).mean(-1, keepdim=True) + eps)
        y = src * inv.float()
        if weight is not None:
            y = y * weight.float()
        out.copy_(y.to(out.dtype))

    def gemm(self, a, w, out, accumulate=False, then_norm=None):
        self.calls.append("gemm")
        product = (a.double() @ w.double().t()).float()
        if accumulate:
            product = product + out.float()
        out.copy_(product.to(out.dtype))
        return None         # this double never prepares a following norm: the norm runs as a step of its own

    def qk_norm_rope_cache(self, qkv, q_out, q_weight, k_weight, eps, cos, sin, positions, row_seq,
                           k_pages, v_pages, page_table, n_heads, n_kv_heads, head_dim, write_kv, max_position):
        self.calls.append("qk_norm_rope_cache")
        n_rows = qkv.shape[0]
        q_width, kv_width = n_heads * head_dim, n_kv_heads * head_dim
        q = qkv[:, :q_width].float().reshape(n_rows, n_heads, head_dim)
        k = qkv[:, q_width:q_width + kv_width].float().reshape(n_rows, n_kv_heads, head_dim)
        v = qkv[:, q_width + kv_width:].reshape(n_rows, n_kv_heads, head_dim)

        def norm(x, w):
            if w is None:
                return x
            inv = 1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)
            return x * inv.float() * w.float()

        def rotate(x):
            if cos is None:
                return x
            half = cos.shape[1]
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]
            a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
            return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)

        q_out.copy_(rotate(norm(q, q_weight)).reshape(n_rows, q_width).to(q_out.dtype))
        if not write_kv:
            return
        k = rotate(norm(k, k_weight))
        for row in range(n_rows):
            pos = int(positions[row])
            page = int(page_table[int(row_seq[row]), pos // PAGE])
            k_pages[page, :, pos % PAGE, :] = k[row].to(k_pages.dtype)
            v_pages[page, :, :, pos % PAGE] = v[row].to(v_pages.dtype)

    def attention(self, q, out, k_pages, v_pages, page_table, row_seq, positions, n_heads, n_kv_heads, head_dim,
                  scale, window=0, layout=None, chunk=0, sinks=None):
        self.calls.append("attention")
        assert not (window and chunk)
        n_rows = q.shape[0]
        group = n_heads // n_kv_heads
        qh = q.float().reshape(n_rows, n_heads, head_dim)
        result = torch.empty_like(qh)
        for row in range(n_rows):
            pos, seq = int(positions[row]), int(row_seq[row])
            first = max(0, pos - window + 1) if window else (pos - pos % chunk if chunk else 0)
            index = torch.arange(first, pos + 1)
            pages = page_table[seq, index // PAGE].long()
            keys = k_pages[pages, :, index % PAGE, :].float()      # [n, kv_heads, head_dim]
            values = v_pages[pages, :, :, index % PAGE].float()
            for head in range(n_heads):
                kv = head // group
                scores = (keys[:, kv, :].double() @ qh[row, head].double()).float() * scale
                if sinks is not None:      # one more term in the sum, with no value
                    probs = torch.softmax(torch.cat([scores, sinks[head].float().reshape(1)]), dim=0)[:-1]
                else:
                    probs = torch.softmax(scores, dim=0)
                result[row, head] = (probs.double() @ values[:, kv, :].double()).float()
        out.copy_(result.reshape(n_rows, n_heads * head_dim).to(out.dtype))

    def pack_weight(self, w):
        return w

    # ---- residual streams, kept-apart sublayer results ----
    def streams_open(self, x, out):
        self.calls.append("streams_open")
        out.copy_(x.unsqueeze(1).expand_as(out))

    def streams_rmsnorm(self, x, take, weight, eps, out, rows=None):
        self.calls.append("streams_rmsnorm")
        src = x if rows is None else x[rows.long()]
        share = torch.ones(x.shape[1]) if take is None else take.float()
        u = (src.double() * share.double()[None, :, None]).sum(1).float()
        y = u * (1.0 / torch.sqrt((u.double() ** 2).mean(-1, keepdim=True) + eps)).float()
        if weight is not None:
            y = y * weight.float()
        out.copy_(y.to(out.dtype))

    def streams_update(self, x, y, mix=None, give=None, scale=None):
        self.calls.append("streams_update")
        streams = x.shape[1]
        m = torch.eye(streams, dtype=torch.float64) if mix is None else mix.double()
        g = torch.ones(streams, dtype=torch.float64) if give is None else give.double()
        add = y.double() * (scale.double() if scale is not None else 1.0)
        new = torch.einsum("st,nsd->ntd", m, x.double()) + g[None, :, None] * add[:, None, :]
        x.copy_(new.float())

    def streams_update_rmsnorm(self, x, y, mix, give, scale, take, weight, eps, out):
        self.streams_update(x, y, mix, give, scale)
        self.streams_rmsnorm(x, take, weight, eps, out)

    def scale(self, x, factor):
        self.calls.append("scale")
        x.mul_(factor)

    def relu_squared(self, x, out=None):
        self.calls.append("relu_squared")
        (x if out is None else out).copy_((x.float().clamp(min=0) ** 2).to(x.dtype))

    # ---- linear attention with a decay ----
    def lightning_scan(self, proj, q_off, k_off, v_off, state, decay, seq_start, seq_slot, out, n_heads, dim, vdim,
                       max_rows_per_seq=None):
        self.calls.append("lightning_scan")
        silu = lambda z: z / (1 + torch.exp(-z))
        p = proj.float()
        for b in range(seq_slot.shape[0]):
            lo, hi, slot = int(seq_start[b]), int(seq_start[b + 1]), int(seq_slot[b])
            for row in range(lo, hi):
                q = silu(p[row, q_off:q_off + n_heads * dim]).reshape(n_heads, dim)
                k = silu(p[row, k_off:k_off + n_heads * dim]).reshape(n_heads, dim)
                v = silu(p[row, v_off:v_off + n_heads * vdim]).reshape(n_heads, vdim)
                s = state[slot] * decay.float()[:, None, None] + k[:, :, None] * v[:, None, :]
                state[slot] = s
                out[row] = torch.einsum("hdv,hd->hv", s.double(), q.double()).float().reshape(-1)

    def gated_rmsnorm(self, o, proj, gate_off, weight, eps, out):
        self.calls.append("gated_rmsnorm")
        width = o.shape[1]
        y = o * (1.0 / torch.sqrt((o.double() ** 2).mean(-1, keepdim=True) + eps)).float()
        if weight is not None:
            y = y * weight.float()
        out.copy_((y * torch.sigmoid(proj[:, gate_off:gate_off + width].float())).to(out.dtype))

    # ---- attention over a cached latent ----
    @staticmethod
    def _turn(x, freq, turned, positions, neighbours=False, magnitude=1.0):
        """x [n, ..., w]: the first `turned` of the last axis in pairs (i, i + turned/2), or (2i, 2i + 1) with `neighbours`, by the
        float32 angle position * freq[i]; cosines and sines times `magnitude`."""
        if not turned:
            return x
        half = turned // 2
        angle = (positions.float()[:, None] * freq.float()[None, :]).double()
        shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
        c, s = (torch.cos(angle) * magnitude).reshape(shape).float(), (torch.sin(angle) * magnitude).reshape(shape).float()
        if neighbours:
            out = x.clone()
            a, b = x[..., 0:turned:2], x[..., 1:turned:2]
            out[..., 0:turned:2] = a * c - b * s
            out[..., 1:turned:2] = b * c + a * s
            return out
        a, b, rest = x[..., :half], x[..., half:turned], x[..., turned:]
        return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)

    def latent_write(self, down, offset, weight, eps, freq, turned, positions, row_seq, k_pages, v_pages, page_table,
                     rank, rot_dim, write=True, query=None, query_head=0, query_first=0, source_head=0, source_first=0, n_heads=0,
                     query_source=None, neighbours=False, magnitude=1.0):
        self.calls.append("latent_write")
        if query is not None:
            source = down if query_source is None else query_source
            n = source.shape[0]
            xs = source[:, :n_heads * source_head].float().reshape(n, n_heads, source_head)[:, :, source_first:source_first + rot_dim]
            query[:, :n_heads * query_head].view(n, n_heads, query_head)[:, :, query_first:query_first + rot_dim] = self._turn(
                xs, freq, turned, positions, neighbours, magnitude).to(query.dtype)
        if not write:
            return
        x = down[:, offset:offset + rank + rot_dim].float()
        c = x[:, :rank] * (1.0 / torch.sqrt((x[:, :rank].double() ** 2).mean(-1, keepdim=True) + eps)).float()
        if weight is not None:
            c = c * weight.float()
        key = torch.cat([c, self._turn(x[:, rank:], freq, turned, positions, neighbours, magnitude)], dim=-1)
        value = torch.cat([c, torch.zeros(x.shape[0], rot_dim)], dim=-1)
        for row in range(x.shape[0]):
            pos = int(positions[row])
            page = int(page_table[int(row_seq[row]), pos // PAGE])
            k_pages[page, 0, pos % PAGE, :] = key[row].to(k_pages.dtype)
            v_pages[page, 0, :, pos % PAGE] = value[row].to(v_pages.dtype)

    def heads_linear(self, x, x_head, x_first, w, y, y_head, y_first, n_heads):
        self.calls.append("heads_linear")
        n, n_in, n_out = x.shape[0], w.shape[1], w.shape[2]
        xs = x[:, :n_heads * x_head].reshape(n, n_heads, x_head)[:, :, x_first:x_first + n_in]
        result = torch.einsum("nhi,hio->nho", xs.double(), w.double()).float()
        y[:, :n_heads * y_head].view(n, n_heads, y_head)[:, :, y_first:y_first + n_out] = result.to(y.dtype)

    def rotate_heads(self, x, x_head, x_first, y, y_head, y_first, freq, turned, positions, n_heads, width):
        self.calls.append("rotate_heads")
        n = x.shape[0]
        xs = x[:, :n_heads * x_head].reshape(n, n_heads, x_head)[:, :, x_first:x_first + width].float()
        y[:, :n_heads * y_head].view(n, n_heads, y_head)[:, :, y_first:y_first + width] = \
            self._turn(xs, freq, turned, positions).to(y.dtype)

    # ---- layer norm, casts, caps, the token's side input ----
    def layernorm(self, x, weight, bias, eps, out, rows=None):
        self.calls.append("layernorm")
        src = (x if rows is None else x[rows.long()]).double()
        centred = src - src.mean(-1, keepdim=True)
        y = centred / torch.sqrt((centred ** 2).mean(-1, keepdim=True) + eps) * weight.double()
        if bias is not None:
            y = y + bias.double()
        out.copy_(y.to(out.dtype))

    def cast_concat(self, a, b, out):
        self.calls.append("cast_concat")
        out.copy_((a if b is None else torch.cat([a, b], dim=1)).to(out.dtype))

    def softcap(self, x, cap):
        self.calls.append("softcap")
        x.copy_(cap * torch.tanh(x / cap))

    def rms_scale_add(self, hidden, y, weight, eps):
        self.calls.append("rms_scale_add")
        inv = 1.0 / torch.sqrt((y.double() ** 2).mean(-1, keepdim=True) + eps)
        hidden.add_((y.double() * inv * weight.double()).float())

    def gelu_gate_table(self, gate, tokens, table, first, out, token_src=None, fed_tokens=None):
        self.calls.append("gelu_gate_table")
        z = gate.double()
        g = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        out.copy_((g * table[tokens.long(), first:first + gate.shape[1]].double()).to(out.dtype))

    # ---- a short convolution over time with a state ----
    @staticmethod
    def _region(state, offset, floats):
        return state.reshape(state.shape[0], -1)[:, offset:offset + floats]

    def short_conv(self, u, first, weight, bias, state, state_offset, row_seq, seq_start, seq_slot, out, silu=False):
        self.calls.append("short_conv")
        channels, taps = weight.shape
        for b in range(seq_slot.shape[0]):
            lo, hi, slot = int(seq_start[b]), int(seq_start[b + 1]), int(seq_slot[b])
            rows = u[lo:hi, first:first + channels].double()
            if taps > 1:
                old = self._region(state, state_offset, (taps - 1) * channels)[slot].reshape(taps - 1, channels).double()
                rows = torch.cat([old, rows], dim=0)
            y = sum(rows[j:j + hi - lo] * weight[:, j].double()[None, :] for j in range(taps))
            if bias is not None:
                y = y + bias.double()[None, :]
            if silu:
                y = y / (1 + torch.exp(-y))
            out[lo:hi] = y.float()

    def short_conv_state(self, u, first, channels, taps, state, state_offset, seq_start, seq_slot):
        self.calls.append("short_conv_state")
        if taps == 1:
            return
        region = self._region(state, state_offset, (taps - 1) * channels)
        for b in range(seq_slot.shape[0]):
            lo, hi, slot = int(seq_start[b]), int(seq_start[b + 1]), int(seq_slot[b])
            both = torch.cat([region[slot].reshape(taps - 1, channels), u[lo:hi, first:first + channels].float()], dim=0)
            region[slot] = both[-(taps - 1):].reshape(-1)

    # ---- attention normed over the whole projection ----
    def whole_norm_rope_write(self, qkv, q_weight, k_weight, eps, freq, turned, positions, row_seq, q_out, k_pages, v_pages,
                              page_table, n_heads, n_kv_heads, dim, vdim, pad, write_kv):
        self.calls.append("whole_norm_rope_write")
        n = qkv.shape[0]
        q_width, k_width = n_heads * dim, n_kv_heads * dim
        rms = lambda x, w: (x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * w.double())
        q = rms(qkv[:, :q_width], q_weight).reshape(n, n_heads, dim)
        k = rms(qkv[:, q_width:q_width + k_width], k_weight).reshape(n, n_kv_heads, dim)
        v = qkv[:, q_width + k_width:].reshape(n, n_kv_heads, vdim)

        def turn(x):
            if not turned:
                return x
            angles = (positions.float()[:, None] * freq.float()[None, :]).double()[:, None, :]
            cos, sin = torch.cos(angles), torch.sin(angles)
            out = x.clone()
            a, b = x[..., 0:turned:2], x[..., 1:turned:2]
            out[..., 0:turned:2] = a * cos - b * sin
            out[..., 1:turned:2] = b * cos + a * sin
            return out

        wide = torch.zeros(n, n_heads, pad, dtype=torch.float64)
        wide[..., :dim] = turn(q)
        q_out.copy_(wide.reshape(n, n_heads * pad).to(q_out.dtype))
        if not write_kv:
            return
        k = turn(k)
        for row in range(n):
            pos, seq = int(positions[row]), int(row_seq[row])
            page = int(page_table[seq, pos // PAGE])
            k_pages[page, :, pos % PAGE, :] = 0
            v_pages[page, :, :, pos % PAGE] = 0
            k_pages[page, :, pos % PAGE, :dim] = k[row].to(k_pages.dtype)
            v_pages[page, :, :vdim, pos % PAGE] = v[row].to(v_pages.dtype)

    def gate_heads(self, attended, pad, gate, gate_first, out, n_heads, vdim, per_head=False):
        self.calls.append("gate_heads")
        n = attended.shape[0]
        a = attended.float().reshape(n, n_heads, pad)[..., :vdim]
        if gate is None:
            out.copy_(a.reshape(n, n_heads * vdim).to(out.dtype))
        elif per_head:
            out.copy_((a * torch.sigmoid(gate[:, gate_first:gate_first + n_heads].float())[:, :, None]).reshape(n, n_heads * vdim).to(out.dtype))
        else:
            out.copy_((a.reshape(n, n_heads * vdim) * torch.sigmoid(gate[:, gate_first:gate_first + n_heads * vdim].float())).to(out.dtype))

    # ---- norm behind the sum, GELU, heads normed one by one, a matrix memory ----
    def sum_layernorm(self, hidden, y, alpha, weight, bias, eps, rounded=None):
        self.calls.append("sum_layernorm")
        total = alpha * hidden.double() + y.double()
        centred = total - total.mean(-1, keepdim=True)
        result = centred / torch.sqrt((centred ** 2).mean(-1, keepdim=True) + eps) * weight.double()
        if bias is not None:
            result = result + bias.double()
        hidden.copy_(result.float())
        if rounded is not None:
            rounded.copy_(result.to(rounded.dtype))

    def gelu_tanh(self, x, out=None):
        self.calls.append("gelu_tanh")
        z = x.double()
        (x if out is None else out).copy_((0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))).to(x.dtype))

    def head_norm_rope_write(self, proj, first, bias, q_weight, k_weight, eps, freq, turned, positions, row_seq, q_out, k_pages,
                             v_pages, page_table, n_heads, n_kv_heads, dim, vdim, pad, write_kv, neighbours=False, magnitude=1.0):
        self.calls.append("head_norm_rope_write")
        n = proj.shape[0]
        q_width, k_width, v_width = n_heads * dim, n_kv_heads * dim, n_kv_heads * vdim
        x = proj[:, first:first + q_width + k_width + v_width].float()
        if bias is not None:
            x = x + bias.float()
        q = x[:, :q_width].reshape(n, n_heads, dim)
        k = x[:, q_width:q_width + k_width].reshape(n, n_kv_heads, dim)
        v = x[:, q_width + k_width:].reshape(n, n_kv_heads, vdim)
        if q_weight is not None:
            rms = lambda t, w: (t.double() / torch.sqrt((t.double() ** 2).mean(-1, keepdim=True) + eps) * w.double()).float()
            q, k = rms(q, q_weight), rms(k, k_weight)
        q, k = self._turn(q, freq, turned, positions, neighbours, magnitude), self._turn(k, freq, turned, positions, neighbours, magnitude)
        wide = torch.zeros(n, n_heads, pad)
        wide[..., :dim] = q
        q_out.copy_(wide.reshape(n, n_heads * pad).to(q_out.dtype))
        if not write_kv:
            return
        for row in range(n):
            pos, seq = int(positions[row]), int(row_seq[row])
            page = int(page_table[seq, pos // PAGE])
            k_pages[page, :, pos % PAGE, :] = 0
            v_pages[page, :, :, pos % PAGE] = 0
            k_pages[page, :, pos % PAGE, :dim] = k[row].to(k_pages.dtype)
            v_pages[page, :, :vdim, pos % PAGE] = v[row].to(v_pages.dtype)

    MLSTM_BESIDE = 4

    @staticmethod
    def mlstm_state_floats(n_heads, dim, vdim):
        return n_heads * ((vdim + 1) * dim + 1)

    def mlstm_gates(self, pre, bias, cap, state, seq_start, seq_slot, beside, n_heads, dim, vdim):
        self.calls.append("mlstm_gates")
        x = pre.float() + (bias.float() if bias is not None else 0.0)
        gate_i = cap * torch.tanh(x[:, :n_heads] / cap)
        gate_f = torch.nn.functional.logsigmoid(cap * torch.tanh(x[:, n_heads:] / cap))
        head_floats = (vdim + 1) * dim + 1
        out = beside.view(-1, n_heads, 4)
        for b in range(seq_slot.shape[0]):
            slot = int(seq_slot[b])
            m = state[slot].view(n_heads, head_floats)[:, -1].clone()
            for row in range(int(seq_start[b]), int(seq_start[b + 1])):
                new = torch.maximum(gate_f[row] + m, gate_i[row])
                out[row, :, 0] = torch.exp(gate_f[row] + m - new)
                out[row, :, 1] = torch.exp(gate_i[row] - new)
                out[row, :, 2] = new
                m = new
            state[slot].view(n_heads, head_floats)[:, -1] = m

    def mlstm_scan(self, proj, q_off, k_off, v_off, beside, state, seq_start, seq_slot, read, n_heads, dim, vdim):
        self.calls.append("mlstm_scan")
        n = proj.shape[0]
        q = proj[:, q_off:q_off + n_heads * dim].float().reshape(n, n_heads, dim) * (1.0 / (dim ** 0.5))
        k = proj[:, k_off:k_off + n_heads * dim].float().reshape(n, n_heads, dim)
        v = torch.cat([proj[:, v_off:v_off + n_heads * vdim].float().reshape(n, n_heads, vdim), torch.ones(n, n_heads, 1)], dim=-1)
        head_floats = (vdim + 1) * dim + 1
        factors = beside.view(n, n_heads, 4)
        for b in range(seq_slot.shape[0]):
            slot = int(seq_slot[b])
            held = state[slot].view(n_heads, head_floats)[:, :-1].reshape(n_heads, vdim + 1, dim)      # column-major: [column][dim]
            S = held.clone().double()
            for row in range(int(seq_start[b]), int(seq_start[b + 1])):
                a, w = factors[row, :, 0].double(), factors[row, :, 1].double()
                S = a[:, None, None] * S + w[:, None, None] * v[row].double()[:, :, None] * k[row].double()[:, None, :]
                got = torch.einsum("hcd,hd->hc", S, q[row].double()).float()
                read[row] = got[:, :vdim].reshape(-1)
                factors[row, :, 3] = got[:, vdim]
                S = S.float().double()
            state[slot].view(n_heads, head_floats)[:, :-1] = S.float().reshape(n_heads, -1)

    def mlstm_finish(self, read, beside, proj, gate_off, weight, eps, out, n_heads, vdim):
        self.calls.append("mlstm_finish")
        n = read.shape[0]
        factors = beside.view(n, n_heads, 4)
        under = torch.maximum(factors[:, :, 3].abs(), torch.exp(-factors[:, :, 2])) + 1e-6
        o = read.view(n, n_heads, vdim).double() / under.double()[:, :, None]
        o = (o / torch.sqrt((o ** 2).mean(-1, keepdim=True) + eps)).reshape(n, n_heads * vdim)
        if weight is not None:
            o = o * weight.double()
        gate = torch.sigmoid(proj[:, gate_off:gate_off + n_heads * vdim].double())
        out.copy_((o * gate).to(out.dtype))

    # ---- a state-space recurrence ----
    def ssm_scan(self, xbc, proj, dt_first, dt_bias, a_log, d_skip, state, state_offset, seq_start, seq_slot, out, n_heads, vdim,
                 n_state, n_groups, max_rows_per_seq=None):
        self.calls.append("ssm_scan")
        inner, per = n_heads * vdim, n_heads // n_groups
        region = self._region(state, state_offset, n_heads * n_state * vdim)
        rate = torch.exp(a_log.double())
        for b in range(seq_slot.shape[0]):
            lo, hi, slot = int(seq_start[b]), int(seq_start[b + 1]), int(seq_slot[b])
            s = region[slot].reshape(n_heads, n_state, vdim).double()
            for row in range(lo, hi):
                x = xbc[row, :inner].double().reshape(n_heads, vdim)
                bm = xbc[row, inner:inner + n_groups * n_state].double().reshape(n_groups, n_state).repeat_interleave(per, dim=0)
                cm = xbc[row, inner + n_groups * n_state:].double().reshape(n_groups, n_state).repeat_interleave(per, dim=0)
                dt = torch.nn.functional.softplus(proj[row, dt_first:dt_first + n_heads].double() + dt_bias.double(), threshold=40.0)
                s = (torch.exp(-rate * dt)[:, None, None] * s + (dt[:, None] * bm)[:, :, None] * x[:, None, :]).float().double()
                out[row] = (torch.einsum("hnv,hn->hv", s, cm) + d_skip.double()[:, None] * x).float().reshape(-1)
            region[slot] = s.float().reshape(-1)

    def gated_group_rmsnorm(self, y, z, z_first, weight, eps, out, groups, gate_after=False):
        self.calls.append("gated_group_rmsnorm")
        n, width = y.shape
        g = z[:, z_first:z_first + width].double()
        gate = g / (1 + torch.exp(-g))
        v = (y.double() if gate_after else y.double() * gate).reshape(n, groups, width // groups)
        v = (v / torch.sqrt((v ** 2).mean(-1, keepdim=True) + eps)).reshape(n, width)
        out.copy_((v * weight.double() * (gate if gate_after else 1.0)).to(out.dtype))

    # ---- routed experts ----
    @staticmethod
    def _clamped_glu(g, u, limit, alpha, shift=1.0):
        g, u = g.clamp(max=limit), u.clamp(min=-limit, max=limit)
        return g * torch.sigmoid(alpha * g) * (u + shift)

    def route_top_k(self, logits, bias, chosen, weights, scoring="softmax"):
        self.calls.append("route_top_k")
        z = logits.double() + (bias.double() if bias is not None else 0.0)
        order = torch.argsort(-z, dim=-1, stable=True)[:, :chosen.shape[1]]
        chosen.copy_(order.to(torch.int32))
        picked = torch.gather(z, 1, order)
        weights.copy_((torch.sigmoid(picked) if scoring == "sigmoid" else torch.softmax(picked, dim=-1)).float())

    def experts_gate_up(self, h, chosen, w_gate_up, inner, limit, alpha, shift=1.0, in_weights=None):
        self.calls.append("experts_gate_up")
        top, ff = chosen.shape[1], w_gate_up.shape[1] // 2
        for row in range(h.shape[0]):
            for j in range(top):
                both = w_gate_up[int(chosen[row, j])].double() @ h[row].double()
                if in_weights is not None:
                    both = both * float(in_weights[row, j])
                inner[row * top + j] = self._clamped_glu(both[:ff], both[ff:], limit, alpha, shift).to(inner.dtype)

    def experts_down(self, inner, chosen, weights, w_down, hidden):
        self.calls.append("experts_down")
        top = chosen.shape[1]
        for row in range(hidden.shape[0]):
            total = torch.zeros(hidden.shape[1], dtype=torch.float64)
            for j in range(top):
                total += (float(weights[row, j]) if weights is not None else 1.0) * (w_down[int(chosen[row, j])].double() @ inner[row * top + j].double())
            hidden[row] += total.float()

    def experts_group(self, chosen, lists, counts):
        self.calls.append("experts_group")
        flat = chosen.reshape(-1)
        for e in range(counts.shape[0]):
            found = torch.nonzero(flat == e).reshape(-1).to(torch.int32)
            counts[e] = found.numel()
            lists[e, :found.numel()] = found

    def experts_rows_take(self, inputs):
        return inputs % 8 == 0

    def experts_rows(self, rows, rows_per_pair_row, lists, counts, w, out, gated=False, limit=0.0, alpha=0.0, shift=1.0, in_weights=None):
        self.calls.append("experts_rows")
        for e in range(counts.shape[0]):
            for pair in lists[e, :int(counts[e])].tolist():
                result = w[e].double() @ rows[pair // rows_per_pair_row].double()
                if gated:
                    half = result.shape[0] // 2
                    if in_weights is not None:
                        result = result * float(in_weights.reshape(-1)[pair])
                    result = self._clamped_glu(result[:half], result[half:], limit, alpha, shift)
                out[pair] = result.to(out.dtype)

    def experts_gather(self, x, top, lists, counts, offsets, gathered, place, in_weights=None):
        self.calls.append("experts_gather")
        for e in range(counts.shape[0]):
            for i, pair in enumerate(lists[e, :int(counts[e])].tolist()):
                row = x[pair // top]
                gathered[int(offsets[e]) + i] = row if in_weights is None else (row.float() * in_weights.reshape(-1)[pair]).to(x.dtype)
                place[pair] = int(offsets[e]) + i

    def experts_combine(self, y, place, weights, hidden, top=None):
        self.calls.append("experts_combine")
        n, top = weights.shape if weights is not None else (hidden.shape[0], int(top))
        index = (place if place is not None else torch.arange(n * top)).long().reshape(n, top)
        share = weights.double()[:, :, None] if weights is not None else 1.0
        hidden.add_((share * y.double()[index]).sum(1).float())

    def clamped_glu(self, gate_up, out, limit, alpha, shift=1.0):
        self.calls.append("clamped_glu")
        ff = out.shape[1]
        out.copy_(self._clamped_glu(gate_up[:, :ff].double(), gate_up[:, ff:].double(), limit, alpha, shift).to(out.dtype))

    # ---- gated linear attention, a norm over a slice, a weighted sum ----
    def gla_scan(self, proj, q_off, k_off, v_off, z, bias, tau, q_scale, state, seq_start, seq_slot, out, n_heads, dim, vdim,
                 max_rows_per_seq=None):
        self.calls.append("gla_scan")
        kw, vw = n_heads * dim, n_heads * vdim
        log_alpha = torch.nn.functional.logsigmoid(z.double() + bias.double()) / tau
        for s in range(seq_slot.shape[0]):
            slot = int(seq_slot[s])
            memory = state[slot].double()
            for row in range(int(seq_start[s]), int(seq_start[s + 1])):
                q = proj[row, q_off:q_off + kw].double().reshape(n_heads, dim) * q_scale
                key = proj[row, k_off:k_off + kw].double().reshape(n_heads, dim)
                value = proj[row, v_off:v_off + vw].double().reshape(n_heads, vdim)
                memory = torch.exp(log_alpha[row]).reshape(n_heads, dim, 1) * memory + key[:, :, None] * value[:, None, :]
                memory = memory.float().double()      # the state is a float32
                out[row] = torch.einsum("hdv,hd->hv", memory, q).float().reshape(-1)
            state[slot] = memory.float()

    def slice_rmsnorm(self, x, first, weight, eps, out):
        self.calls.append("slice_rmsnorm")
        v = x[:, first:first + out.shape[1]].double()
        out.copy_((v / torch.sqrt((v ** 2).mean(-1, keepdim=True) + eps) * weight.double()).to(out.dtype))

    def weighted_sum(self, out, x, a, y, b):
        self.calls.append("weighted_sum")
        out.copy_((a * x.double() + b * y.double()).float())

    def gemm_swiglu(self, a, w, out):
        self.calls.append("gemm_swiglu")
        both = torch.empty(a.shape[0], w.shape[0], dtype=a.dtype)
        self.gemm(a, w, both)
        self.swiglu(both, out)

    def swiglu(self, gate_up, out):
        self.calls.append("swiglu")
        width = out.shape[1]
        g, u = gate_up[:, :width].float(), gate_up[:, width:].float()
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))

    def sample(self, logits, tokens, bad, temperature=None, top_k=None, top_p=None, uniform=None):
        self.calls.append("sample")
        for row in range(logits.shape[0]):
            x = logits[row]
            if not torch.isfinite(x).all():
                tokens[row], bad[row] = -1, 1
                continue
            bad[row] = 0
            temp = float(temperature[row]) if temperature is not None else 0.0
            if temp <= 0:
                tokens[row] = int(torch.argmax(x))
                continue
            keep = torch.ones_like(x, dtype=torch.bool)
            k = int(top_k[row]) if top_k is not None else 0
            if 0 < k < x.numel():
                keep &= x >= torch.topk(x, k).values[-1]
            e = torch.where(keep, torch.exp((x - x.max()) / temp), torch.zeros_like(x)).double()
            p = float(top_p[row]) if top_p is not None else 1.0
            if 0 < p < 1:
                order = torch.argsort(e, descending=True)
                mass = torch.cumsum(e[order], 0)
                count = int(torch.searchsorted(mass, p * e.sum()).clamp(max=x.numel() - 1)) + 1
                keep &= e >= e[order][count - 1]
                e = torch.where(keep, e, torch.zeros_like(e))
            cdf = torch.cumsum(e, 0)
            target = float(uniform[row]) * float(cdf[-1])
            tokens[row] = int(torch.searchsorted(cdf, torch.tensor(target, dtype=cdf.dtype), right=True)
                              .clamp(max=x.numel() - 1))
