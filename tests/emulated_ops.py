"""A host stand-in for the kernel library, for tests only.

It implements the kernel library's Python interface (``prefixserve_amd.kernels.ops.HipOps``)
with plain torch on the CPU, reading and writing the same buffers in the same layouts, so
that everything on the host side of a step (batch packing, block tables, page reuse, the
scheduler, replay) can be tested without a GPU. The package itself never uses it: without
the compiled kernels and a GPU the engine raises.
"""

from __future__ import annotations

import contextlib

import torch

PAGE = 16


class EmulatedOps:
    PREFILL_TILE_Q = 64
    name = "emulated"

    def __init__(self, device: torch.device | str = "cpu", workspace=None) -> None:
        self.device = torch.device(device)
        self.ws = workspace

    def step_scope(self):
        return contextlib.nullcontext()

    def prepare_matrix(self, w: torch.Tensor, rt) -> torch.Tensor:
        return w.to(device=rt.device, dtype=rt.dtype).contiguous()

    def embed(self, ids, table, out) -> None:
        out.copy_(table[ids.long()].float())

    def add_rmsnorm(self, residual, delta, weight, eps, out) -> None:
        if delta is not None:
            residual.add_(delta.float())
        x = residual
        out.copy_((weight.float() * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)).to(out.dtype))

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps, out) -> None:
        x = residual[rows.long()]
        if delta is not None:
            x = x + (delta[:, rows.long()].float().sum(0) if delta.dim() == 3 else delta[rows.long()].float())
        out.copy_((weight.float() * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)).to(out.dtype))

    def linear(self, x, w, out) -> None:
        out.copy_((x.float() @ w.float().T).to(out.dtype))

    def linear_to_residual(self, x, w, name, residual=None):
        out = self.ws.get(name, (x.shape[0], w.shape[0]), x.dtype)
        self.linear(x, w, out)
        return out

    def linear_swiglu(self, x, w_gate_up, out, activation="silu") -> None:
        gu = x.float() @ w_gate_up.float().T
        inter = gu.shape[1] // 2
        act = {"silu": torch.nn.functional.silu, "relu": torch.relu,
               "gelu_tanh": lambda z: torch.nn.functional.gelu(z, approximate="tanh")}[activation]
        out.copy_((act(gu[:, :inter]) * gu[:, inter:]).to(out.dtype))

    def residual_add(self, residual, delta) -> None:
        residual.add_(delta.float().sum(0) if delta.dim() == 3 else delta.float())

    def stream_affine(self, x, factor=1.0, row=None) -> None:
        x.mul_(factor)
        if row is not None:
            x.add_(row)

    def concat_to_activation(self, a, b, out) -> None:
        out.copy_(torch.cat([a, b], dim=-1).to(out.dtype))

    def heads_linear(self, x, x_offset, x_head, w, out, out_offset, out_head) -> None:
        heads, n, k = w.shape
        for h in range(heads):
            xs = x[:, x_offset + h * x_head: x_offset + h * x_head + k].float()
            out[:, out_offset + h * out_head: out_offset + h * out_head + n] = (xs @ w[h].float().T).to(out.dtype)

    def latent_kv_append(self, rows, q_lat, hq, dim, rot, rank, slots, positions, table, norm_weight, eps, kv, write_slot) -> None:
        t = rows.shape[0]
        low = rows[:, hq * (dim + rot):].float()
        c = low[:, :rank]
        c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * norm_weight

        def turn(v):                                       # [..., rot], neighbours paired
            cs = table[positions.long()]                   # [t, rot/2, 2]
            while cs.dim() - 1 < v.dim():
                cs = cs.unsqueeze(1)
            a, b = v[..., 0::2], v[..., 1::2]
            res = torch.empty_like(v)
            res[..., 0::2] = a * cs[..., 0] - b * cs[..., 1]
            res[..., 1::2] = b * cs[..., 0] + a * cs[..., 1]
            return res

        key = torch.zeros((t, slots))
        key[:, :rank] = c
        if rot:
            key[:, rank: rank + rot] = turn(low[:, rank: rank + rot])
        val = torch.zeros((t, slots))
        val[:, :rank] = c
        if kv is not None:
            page, off = (write_slot // PAGE).long(), (write_slot % PAGE).long()
            kv[:, 0].view(kv.shape[0], 1, PAGE, slots)[page, 0, off, :] = key.to(kv.dtype)
            kv[:, 1].view(kv.shape[0], 1, slots, PAGE)[page, 0, :, off] = val.to(kv.dtype)
        q = rows[:, : hq * (dim + rot)].view(t, hq, dim + rot).float()
        ql = q_lat.view(t, hq, slots)
        ql[:, :, rank:] = 0
        if rot:
            ql[:, :, rank: rank + rot] = turn(q[:, :, dim:]).to(q_lat.dtype)

    def causal_conv(self, rows, col, bias, conv_w, conv_b, u, state, ctx) -> None:
        width, taps = conv_w.shape
        starts = ctx.item_start.tolist()
        for i in range(ctx.num_items):
            t0, t1 = starts[i], starts[i + 1]
            slot = int(ctx.slots[i])
            saved = state[slot, : (taps - 1) * width].view(taps - 1, width)
            v = torch.cat([saved, rows[t0:t1, col: col + width].float() + bias], dim=0)
            acc = conv_b.expand(t1 - t0, width).clone()
            for j in range(taps):
                acc += conv_w[:, j] * v[j: j + t1 - t0]
            u[t0:t1] = acc

    def gated_scan(self, gates, gate_bias, u, decay, rows, y_col, x_col, y_bias, x_bias, out, state, ctx, blocks, taps) -> None:
        t, width = u.shape
        bw = width // blocks
        g = gates.view(t, blocks, 2 * bw) + gate_bias.view(blocks, 2 * bw)
        r = torch.sigmoid(g[:, :, :bw]).reshape(t, width)
        gi = torch.sigmoid(g[:, :, bw:]).reshape(t, width)
        la = decay * r
        a, step = torch.exp(la), torch.sqrt(-torch.expm1(2 * la))
        y = torch.nn.functional.gelu(rows[:, y_col: y_col + width].float() + y_bias, approximate="tanh")
        starts = ctx.item_start.tolist()
        for i in range(ctx.num_items):
            t0, t1 = starts[i], starts[i + 1]
            slot = int(ctx.slots[i])
            s = state[slot, (taps - 1) * width:].clone()
            for k in range(t0, t1):
                s = a[k] * s + step[k] * gi[k] * u[k]
                out[k] = (s * y[k]).to(out.dtype)
            state[slot, (taps - 1) * width:] = s
            if taps > 1:
                saved = state[slot, : (taps - 1) * width].view(taps - 1, width)
                v = torch.cat([saved, rows[t0:t1, x_col: x_col + width].float() + x_bias], dim=0)
                state[slot, : (taps - 1) * width] = v[-(taps - 1):].reshape(-1)

    def qkv_rope_append(self, x, w_qkv, qkv, hq, hkv, d, positions, table, kv, write_slot) -> None:
        self.linear(x, w_qkv, qkv)
        self.rope_kv_append(qkv, hq, hkv, d, positions, table, kv, write_slot)

    def rope_kv_append(self, qkv, hq, hkv, d, positions, table, kv, write_slot) -> None:
        t = qkv.shape[0]
        q = qkv[:, : hq * d].view(t, hq, d)
        k = qkv[:, hq * d: (hq + hkv) * d].view(t, hkv, d)
        v = qkv[:, (hq + hkv) * d:].view(t, hkv, d)
        if table is not None:
            cs = table[positions.long()]  # [t, d/2, 2]
            cos, sin = cs[..., 0][:, None, :], cs[..., 1][:, None, :]
            for x in (q, k):
                x1, x2 = x[..., : d // 2].float().clone(), x[..., d // 2:].float().clone()
                x[..., : d // 2] = (x1 * cos - x2 * sin).to(x.dtype)
                x[..., d // 2:] = (x2 * cos + x1 * sin).to(x.dtype)
        if kv is not None:
            page = (write_slot // PAGE).long()
            off = (write_slot % PAGE).long()
            kpages = kv[:, 0].view(kv.shape[0], hkv, PAGE, d)
            vpages = kv[:, 1].view(kv.shape[0], hkv, d, PAGE)
            kpages[page, :, off, :] = k
            vpages[page, :, :, off] = v

    def normed(self, x, name="normed.x"):
        return x

    def to_activation(self, src, out) -> None:
        out.copy_(src.to(out.dtype))

    def scaled_add_rmsnorm(self, residual, delta, alpha, weight, eps, out) -> None:
        x = residual * alpha
        if delta is not None:
            x = x + (delta.float().sum(0) if delta.dim() == 3 else delta.float())
        y = weight.float() * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
        residual.copy_(y)
        if out is not None:
            out.copy_(y.to(out.dtype))

    def rope_norm_kv_append(self, qkv, hq, hkv, d, positions, table, kv, write_slot, norm_dim, norm_eps, bias=None,
                            q_weight=None, k_weight=None, values_from_keys=False, q_weight_per_head=False) -> None:
        t = qkv.shape[0]
        heads = qkv[:, : (hq + hkv) * d].view(t, hq + hkv, d)
        x = heads.float()
        if bias is not None:
            x = x + bias.view(hq + hkv, d)
        raw_keys = x[:, hq:].to(qkv.dtype)
        if table is not None:
            cs = table[positions.long()]
            cos, sin = cs[..., 0][:, None, :], cs[..., 1][:, None, :]
            x1, x2 = x[..., : d // 2], x[..., d // 2:]
            x = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
        if norm_dim:
            x = x * torch.rsqrt((x * x).sum(-1, keepdim=True) / norm_dim + norm_eps)
        if q_weight is not None:
            x[:, :hq] = x[:, :hq] * (q_weight.view(hq, d) if q_weight_per_head else q_weight)
        if k_weight is not None:
            x[:, hq:] = x[:, hq:] * k_weight
        heads.copy_(x.to(qkv.dtype))
        if kv is not None:
            page, off = (write_slot // PAGE).long(), (write_slot % PAGE).long()
            kv[:, 0].view(kv.shape[0], hkv, PAGE, d)[page, :, off, :] = heads[:, hq:]
            vals = raw_keys if values_from_keys else qkv[:, (hq + hkv) * d:].view(t, hkv, d)
            kv[:, 1].view(kv.shape[0], hkv, d, PAGE)[page, :, :, off] = vals

    def moe_route(self, x, w_router, chosen, weight, w_router_act=None, bias=None, mode=0) -> None:
        z = x.float() @ w_router.float().T
        if bias is not None:
            z = z + bias
        s = torch.sigmoid(z) if mode == 0 else z
        order = torch.argsort(-s, dim=-1, stable=True)[:, : chosen.shape[1]]
        chosen.copy_(order.to(torch.int32))
        picked = torch.gather(s, 1, order)
        weight.copy_(picked if mode == 0 else torch.softmax(picked, dim=-1))

    def moe_experts(self, x, chosen, weight, w_gate_up, w_down, act, out, gate_alpha, limit, up_shift,
                    weight_on_output=False) -> None:
        t, k = chosen.shape
        f = w_gate_up.shape[1] // 2
        for i in range(t):
            for j in range(k):
                e = int(chosen[i, j])
                h = x[i].float() * (1.0 if weight_on_output else weight[i, j])
                gu = w_gate_up[e].float() @ h
                g, u = gu[:f].clamp(max=limit), gu[f:].clamp(-limit, limit)
                y = (g * torch.sigmoid(gate_alpha * g) * (u + up_shift)).to(act.dtype)
                act[i * k + j] = y
                out[j, i] = (w_down[e].float() @ y.float()) * (weight[i, j] if weight_on_output else 1.0)

    def row_gate(self, out, x, w) -> None:
        out.mul_(torch.sigmoid(x.float() @ w)[:, None])

    def layernorm_step(self, residual, delta, post, pre, out, rows=None) -> None:
        def ln(y, terms):
            w, b, eps = terms
            d = y - y.mean(-1, keepdim=True)
            return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w + b

        if delta is not None:
            residual.add_(ln(delta.float().sum(0) if delta.dim() == 3 else delta.float(), post))
        if out is not None:
            out.copy_(ln(residual if rows is None else residual[rows.long()], pre).to(out.dtype))

    def add_sinusoid(self, x, positions, freq) -> None:
        h = x.shape[1]
        ang = positions.double()[:, None] * freq[torch.arange(h) // 2][None, :]
        x.add_(torch.where(torch.arange(h) % 2 == 0, torch.sin(ang), torch.cos(ang)).float())

    def short_conv(self, rows, col, conv_w, out, state, state_offset, ctx, silu=True, bias=None) -> None:
        channels, taps = conv_w.shape
        keep = taps - 1
        starts = ctx.item_start.tolist()
        for i in range(ctx.num_items):
            t0, t1 = starts[i], starts[i + 1]
            saved = state[int(ctx.slots[i]), state_offset: state_offset + keep * channels].view(keep, channels)
            v = torch.cat([saved, rows[t0:t1, col: col + channels].float()], dim=0)
            acc = torch.zeros((t1 - t0, channels)) if bias is None else bias.expand(t1 - t0, channels).clone()
            for j in range(taps):
                acc += conv_w[:, j] * v[j: j + t1 - t0]
            out[t0:t1] = (torch.nn.functional.silu(acc) if silu else acc).to(out.dtype)
            if keep:
                saved.copy_(v[-keep:].clone())

    def gated_delta_prepare(self, u, groups, dim, gates, decay_log, decay_bias, coef, q_scale, unit_eps) -> None:
        t, heads = u.shape[0], decay_log.numel()
        qk = u[:, : 2 * groups * dim].view(t, 2 * groups, dim)
        unit = qk * torch.rsqrt((qk * qk).sum(-1, keepdim=True) + unit_eps)
        unit[:, :groups] *= q_scale
        qk.copy_(unit)
        b = torch.sigmoid(gates[:, :heads])
        g = torch.exp(-torch.exp(decay_log) * torch.nn.functional.softplus(gates[:, heads:] + decay_bias))
        coef.copy_(torch.cat([g, -b, b], dim=-1))

    def general_delta_prepare(self, rows, r_col, k_col, v_col, a_col, l_col, rate_bias, decay_out, decay_bias, operands,
                              heads, dim, decay_floor, unit_eps) -> None:
        t, hd = rows.shape[0], heads * dim
        r, k, v, a = (rows[:, c: c + hd].float() for c in (r_col, k_col, v_col, a_col))
        low = torch.tanh(rows[:, l_col: l_col + decay_out.shape[0]].float()) @ decay_out + decay_bias
        w = torch.exp(-decay_floor * torch.sigmoid(low))
        kh = k.view(t, heads, dim)
        c = (kh * torch.rsqrt((kh * kh).sum(-1, keepdim=True) + unit_eps)).reshape(t, hd)
        operands.copy_(torch.cat([r, k, v, w, -torch.sigmoid(a + rate_bias) * c, c], dim=-1))

    def delta_scan(self, keys, directions, removals, queries, key_groups, decay_vectors, decay, removal_scale,
                   value_scale, values, out, state, state_offset, ctx, heads, dim, vdim, reads_decayed, no_removal=False) -> None:
        t = out.shape[0]

        def vec(pair, n, size):
            return pair[0][:, pair[1]: pair[1] + n * size].view(t, n, size)

        def num(pair):
            return torch.ones((t, heads)) if pair is None else pair[0][:, pair[1]: pair[1] + heads]

        rep = heads // key_groups
        kk, cc, pp, rr = (vec(p, key_groups, dim).repeat_interleave(rep, dim=1) for p in (keys, directions, removals, queries))
        dv = torch.ones((t, heads, dim)) if decay_vectors is None else vec(decay_vectors, heads, dim)
        ds, ps, xs = num(decay), num(removal_scale), num(value_scale)
        xx = vec(values, heads, vdim)
        o = out.view(t, heads, vdim)
        starts = ctx.item_start.tolist()
        for i in range(ctx.num_items):
            st = state[int(ctx.slots[i]), state_offset: state_offset + heads * vdim * dim].view(heads, vdim, dim)
            s = st.clone().transpose(1, 2)                                   # [heads, dim, vdim]
            for k in range(starts[i], starts[i + 1]):
                dec = (dv[k] * ds[k][:, None])[:, :, None] * s
                dot = torch.einsum("hd,hdv->hv", cc[k], dec if reads_decayed else s)
                s = dec + (ps[k][:, None] * pp[k])[:, :, None] * dot[:, None, :] \
                    + kk[k][:, :, None] * (xs[k][:, None] * xx[k])[:, None, :]
                o[k] = torch.einsum("hd,hdv->hv", rr[k], s)
            st.copy_(s.transpose(1, 2))

    def heads_norm_gate(self, o, heads, vdim, weight, weight_per_head, eps, gate_rows, gate_col, activation, out) -> None:
        t = o.shape[0]
        y = o.view(t, heads, vdim)
        y = y * torch.rsqrt((y * y).mean(-1, keepdim=True) + eps) * (weight.view(heads, vdim) if weight_per_head else weight)
        z = gate_rows[:, gate_col: gate_col + heads * vdim].float().view(t, heads, vdim)
        act = torch.nn.functional.silu(z) if activation == "silu" else torch.sigmoid(z)
        out.copy_((y * act).reshape(t, heads * vdim).to(out.dtype))

    def expand_kv(self, x, rep):
        """[keys, kv_heads, d] -> [keys, heads, d]: query head h reads kv head h // rep."""
        return x.repeat_interleave(rep, dim=1)

    # ----------------------------------------------- several streams, side-by-side mixers, dense feed-forward

    def stream_rms_norm(self, x, weight, eps) -> None:
        x.copy_(weight * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps))

    def hyper_read(self, streams, read, weight, eps, out, factor=None) -> None:
        u = torch.einsum("s,sth->th", read, streams)
        h = weight.float() * u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps)
        out.copy_((h if factor is None else h * factor).to(out.dtype))

    def hyper_write(self, streams, mix, write, delta, scale=1.0, delta2=None, scale2=0.0) -> None:
        y = scale * (delta.float().sum(0) if delta.dim() == 3 else delta.float())
        if delta2 is not None:
            y = y + scale2 * (delta2.float().sum(0) if delta2.dim() == 3 else delta2.float())
        streams.copy_(torch.einsum("st,sxh->txh", mix, streams) + write[:, None, None] * y[None])

    def weighted_sum(self, a, a_scale, b, b_scale, out) -> None:
        def whole(d):
            return d.float().sum(0) if d.dim() == 3 else d.float()
        out.copy_(a_scale * whole(a) + b_scale * whole(b))

    def activation(self, x, kind) -> None:
        f = {"gelu": torch.nn.functional.gelu, "gelu_tanh": lambda z: torch.nn.functional.gelu(z, approximate="tanh"),
             "silu": torch.nn.functional.silu, "relu": torch.relu}[kind]
        x.copy_(f(x.float()).to(x.dtype))

    def gated_group_norm(self, y, x, x_col, skip, heads, gate_rows, gate_col, weight, groups, eps, out) -> None:
        t, inner = y.shape
        v = y + (skip[:, None] * x[:, x_col: x_col + inner].view(t, heads, inner // heads)).reshape(t, inner)
        g = v * torch.nn.functional.silu(gate_rows[:, gate_col: gate_col + inner].float())
        g = g.view(t, groups, inner // groups)
        g = g * torch.rsqrt((g * g).mean(-1, keepdim=True) + eps)
        out.copy_((g.reshape(t, inner) * weight).to(out.dtype))

    def state_space_prepare(self, dt, dt_bias, decay_log, coef) -> None:
        d = torch.nn.functional.softplus(dt + dt_bias)
        coef.copy_(torch.cat([torch.exp(-torch.exp(decay_log) * d), torch.zeros_like(d), d], dim=-1))

    def matrix_memory_gates(self, gates, gate_bias, cap, coef, state, m_offset, ctx) -> None:
        heads = gates.shape[1] // 2
        starts = ctx.item_start.tolist()
        for i in range(ctx.num_items):
            m = state[int(ctx.slots[i]), m_offset: m_offset + heads]
            for t in range(starts[i], starts[i + 1]):
                z = cap * torch.tanh((gates[t] + gate_bias) / cap)
                il, fl = z[:heads], torch.nn.functional.logsigmoid(z[heads:])
                m_new = torch.maximum(fl + m, il)
                coef[t] = torch.cat([torch.exp(fl + m - m_new), torch.zeros(heads), torch.exp(il - m_new), torch.exp(-m_new)])
                m.copy_(m_new)

    def matrix_memory_operands(self, rows, q_col, k_col, v_col, heads, dim, vdim, q_scale, u, vals) -> None:
        t = rows.shape[0]
        u[:, : heads * dim] = rows[:, q_col: q_col + heads * dim].float() * q_scale
        u[:, heads * dim:] = rows[:, k_col: k_col + heads * dim].float()
        v = vals.view(t, heads, vdim + 1)
        v[:, :, :vdim] = rows[:, v_col: v_col + heads * vdim].float().view(t, heads, vdim)
        v[:, :, vdim] = 1.0

    def memory_read_norm_gate(self, raw, coef, floor_col, heads, vdim, read_eps, weight, eps, gate_rows, gate_col, out) -> None:
        t = raw.shape[0]
        r = raw.view(t, heads, vdim + 1)
        den = torch.maximum(r[:, :, vdim].abs(), coef[:, floor_col: floor_col + heads]) + read_eps
        o = r[:, :, :vdim] / den[:, :, None]
        o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * weight.view(heads, vdim)
        z = gate_rows[:, gate_col: gate_col + heads * vdim].float().view(t, heads, vdim)
        out.copy_((o * torch.sigmoid(z)).reshape(t, heads * vdim).to(out.dtype))

    def pool_kv_append(self, kv, pool_kv, ctx, group, pool_group, hkv, d, block) -> None:
        g, pg = ctx.groups[group], ctx.groups[pool_group]
        offs = g.table_off.tolist()
        for t in range(ctx.num_tokens):
            slot = int(pg.write_slot[t])
            if slot < 0:
                continue
            pos, item = int(ctx.positions[t]), int(ctx.tok_item[t])
            ks, vs = [], []
            for j in range(pos - block + 1, pos + 1):
                page = int(g.block_ids[offs[item] + j // PAGE])
                ks.append(kv[page, 0].view(hkv, PAGE, d)[:, j % PAGE].float())
                vs.append(kv[page, 1].view(hkv, d, PAGE)[:, :, j % PAGE].float())
            pool_kv[slot // PAGE, 0].view(hkv, PAGE, d)[:, slot % PAGE] = torch.stack(ks).mean(0).to(kv.dtype)
            pool_kv[slot // PAGE, 1].view(hkv, d, PAGE)[:, :, slot % PAGE] = torch.stack(vs).mean(0).to(kv.dtype)

    def _masked_attention(self, qkv, out, kv, ctx, group, hq, hkv, d, scale, window, keep_first, pooled, head_gate) -> None:
        g = ctx.groups[group]
        t = qkv.shape[0]
        rep = hq // hkv
        offs = g.table_off.tolist()
        for row in range(t):
            pos, item = int(ctx.positions[row]), int(ctx.tok_item[row])
            seen = [j for j in range(pos + 1) if pos - j < window or j < keep_first]
            keys, vals = [], []
            for j in seen:
                page = int(g.block_ids[offs[item] + j // PAGE])
                keys.append(kv[page, 0].view(hkv, PAGE, d)[:, j % PAGE].float())
                vals.append(kv[page, 1].view(hkv, d, PAGE)[:, :, j % PAGE].float())
            if pooled is not None:
                pkv, pgroup, block = pooled
                pg = ctx.groups[pgroup]
                poffs = pg.table_off.tolist()
                for b in range(max(0, (pos - window + 1) // block)):
                    page = int(pg.block_ids[poffs[item] + b // PAGE])
                    keys.append(pkv[page, 0].view(hkv, PAGE, d)[:, b % PAGE].float())
                    vals.append(pkv[page, 1].view(hkv, d, PAGE)[:, :, b % PAGE].float())
            keys = torch.stack(keys).repeat_interleave(rep, dim=1)          # [n, hq, d]
            vals = torch.stack(vals).repeat_interleave(rep, dim=1)
            q = qkv[row, : hq * d].view(hq, d).float()
            w = torch.softmax(torch.einsum("hd,nhd->hn", q, keys) * scale, dim=-1)
            o = torch.einsum("hn,nhd->hd", w, vals)
            if head_gate is not None:
                o = o * torch.sigmoid(head_gate[row])[:, None]
            out[row] = o.reshape(hq * d).to(out.dtype)

    def paged_attention(self, qkv, out, kv, ctx, group, hq, hkv, d, scale, window, exact_weights=False, sink=None,
                        dist_bias=None, keep_first=0, pooled=None, head_gate=None) -> None:
        if keep_first or pooled is not None or head_gate is not None:
            return self._masked_attention(qkv, out, kv, ctx, group, hq, hkv, d, scale, window, keep_first, pooled, head_gate)
        g = ctx.groups[group]
        t = qkv.shape[0]
        q = qkv[:, : hq * d].view(t, hq, d).float()
        o = out.view(t, hq, d)
        rep = hq // hkv
        starts = ctx.item_start.tolist()
        offs = g.table_off.tolist()
        for i in range(ctx.num_items):
            t0, t1 = starts[i], starts[i + 1]
            pos0, end = int(ctx.item_pos0[i]), int(ctx.item_end[i])
            pages = g.block_ids[offs[i]: offs[i] + -(-end // PAGE)].long()
            keys = kv[pages, 0].view(-1, hkv, PAGE, d).permute(0, 2, 1, 3).reshape(-1, hkv, d)[:end].float()
            vals = kv[pages, 1].view(-1, hkv, d, PAGE).permute(0, 3, 1, 2).reshape(-1, hkv, d)[:end].float()
            keys = self.expand_kv(keys, rep)
            vals = self.expand_kv(vals, rep)
            qi = q[t0:t1].transpose(0, 1)                                  # [hq, n, d]
            scores = torch.matmul(qi, keys.permute(1, 2, 0)) * scale        # [hq, n, end]
            qpos = torch.arange(pos0, end)[:, None]
            kpos = torch.arange(end)[None, :]
            hidden = kpos > qpos
            if window is not None:
                hidden = hidden | (qpos - kpos >= window)
            if dist_bias is not None:
                scores = scores + dist_bias[:, (qpos - kpos).clamp(0, dist_bias.shape[1] - 1)]
            scores = scores.masked_fill(hidden, float("-inf"))
            if sink is not None:
                scores = torch.cat([scores, sink.view(hq, 1, 1).expand(hq, scores.shape[1], 1)], dim=-1)
            probs = torch.softmax(scores, dim=-1)
            if sink is not None:
                probs = probs[..., :-1]
            o[t0:t1] = torch.matmul(probs, vals.transpose(0, 1)).transpose(0, 1).to(out.dtype)

    def argmax(self, logits, out) -> None:
        out.copy_(torch.argmax(logits, dim=-1).to(out.dtype))

    def sample(self, logits, temperatures, uniforms, out) -> None:
        for i in range(logits.shape[0]):
            temp = float(temperatures[i])
            if temp <= 0.0:
                out[i] = int(torch.argmax(logits[i]))
                continue
            z = logits[i].double() / temp
            p = torch.exp(z - z.max())
            c = torch.cumsum(p, 0)
            idx = int(torch.searchsorted(c, float(uniforms[i]) * float(c[-1]), right=True))
            out[i] = min(idx, logits.shape[1] - 1)
