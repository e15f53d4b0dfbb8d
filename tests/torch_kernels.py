"""Plain torch versions of the engine's device operations, one per kernel, with the same
signatures as nano_vllm_amd.kernels.ops.HipKernels.

Two uses, both in tests only: each HIP kernel is compared with its function here, and the
engine's host logic (batching, cache, scheduler) runs on them on the CPU, where no GPU is
present.  The product never imports this file.
"""
from __future__ import annotations

import torch


def _round(x, dtype):
    return x.to(dtype).to(torch.float32)


def v_tile(page_size: int) -> int:
    """Keys per tile of the V cache [pages, kv_heads, page / vt, head_dim, vt]."""
    return 32 if page_size % 32 == 0 else page_size


def new_caches(pages, kv_heads, head_dim, page_size, dtype, device, fill=None, v_head_dim=None):
    """K [pages, kv_heads, page, head_dim] and V [pages, kv_heads, page / vt, v_head_dim, vt]."""
    vt = v_tile(page_size)
    k = torch.zeros((pages, kv_heads, page_size, head_dim), dtype=dtype, device=device)
    v = torch.zeros((pages, kv_heads, page_size // vt, v_head_dim or head_dim, vt), dtype=dtype, device=device)
    if fill is not None:
        k.normal_(0, fill)
        v.normal_(0, fill)
    return k, v


class TorchKernels:
    name = "torch-plain"

    def __init__(self, device="cpu", dtype=torch.float32):
        self.device = torch.device(device)
        self.dtype = dtype
        self.fault_flag = torch.zeros(1, dtype=torch.int32, device=self.device)

    def check_faults(self):
        pass

    # rows
    def embedding(self, table, ids, out=None):
        y = table[ids.long()]
        if out is not None:
            out.copy_(y)
            return out
        return y

    gather_rows = embedding

    def embedding_scaled(self, table, ids, scale):
        return table[ids.long()].float() * scale

    # norms (layernorm.py:16-40)
    def rms_norm(self, x, weight, eps, out=None):
        xf = x.float()
        y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        y = (_round(y, x.dtype) * weight.float()).to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def add_rms_norm(self, x, residual, weight, eps, out=None):
        s = x.float() + residual.float()
        residual.copy_(s.to(x.dtype))
        y = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)
        y = (_round(y, x.dtype) * weight.float()).to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out, residual
        return y, residual

    def stream_rms_norm(self, addends, residual, weight, eps, offset=0.0, out=None):
        """The float32 residual stream takes the sum of the addends; its norm, in float, rounded once."""
        add = None
        dt = out.dtype if out is not None else None
        for a in addends:
            if hasattr(a, "mult"):          # an addend that enters through a norm of its own, times a constant
                x = a.x.float()
                dt = dt or a.x.dtype
                x = a.mult * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + a.eps) * a.weight.float())
            else:
                x = a.float()
                dt = dt or a.dtype
            add = x if add is None else add + x
        if residual is None:
            residual = add.clone()
        elif add is not None:
            residual += add
        y = (residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps) * (offset + weight.float())).to(dt)
        if out is not None:
            out.copy_(y)
            return out, residual
        return y, residual

    def stream_scaled_norm(self, addends, residual, weight, eps, weight2=None, out=None, out2=None, dtype=None):
        """The float32 stream takes every addend times its vector; one or two norms of it, each rounded once."""
        dt = out.dtype if out is not None else dtype
        add = None
        for a, sc in addends:
            dt = a.dtype
            x = a.float() * (sc.float() if sc is not None else 1.0)
            add = x if add is None else add + x
        if residual is None:
            residual = add.clone()
        elif add is not None:
            residual += add
        unit = residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
        y = (unit * weight.float()).to(dt)
        y2 = (unit * weight2.float()).to(dt) if weight2 is not None else None
        if out is not None:
            out.copy_(y)
            y = out
        if out2 is not None and y2 is not None:
            out2.copy_(y2)
            y2 = out2
        return y, y2, residual

    def stream_dyt(self, addends, residual, weight, bias, alpha, out=None):
        """The float32 stream takes the sum of the addends; tanh(alpha * stream) * weight + bias, rounded once."""
        add = None
        for a in addends:
            add = a.float() if add is None else add + a.float()
        if residual is None:
            residual = add.clone()
        elif add is not None:
            residual += add
        dt = addends[0].dtype if addends else out.dtype
        y = (torch.tanh(alpha.float() * residual) * weight.float() + bias.float()).to(dt)
        if out is not None:
            out.copy_(y)
            return out, residual
        return y, residual

    def pair_norm_mean(self, a, wa, b, wb, eps, out=None):
        """Half the sum of the two inputs, each normed over its row with its plain weight."""
        def normed(x, w):
            x = x.float()
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        y = (0.5 * (normed(a, wa) + normed(b, wb))).to(a.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def scale_(self, x, factor):
        return x.mul_(factor)

    @staticmethod
    def _activation(g, act):
        if act == "relu2":
            return torch.relu(g) ** 2
        if act == "relu":
            return torch.relu(g)
        if act == "silu":
            return g * torch.sigmoid(g)
        if act == "gelu_tanh":
            return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
        raise ValueError(act)

    def act(self, x, act="relu2", out=None):
        y = self._activation(x.float(), act).to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    # routed feed-forward
    def moe_route(self, logits, top, group_count, group_keep, scale, routing="sigmoid_groups", bias=None):
        """int32 [T, top] experts and float32 [T, top] weights (scale * sigmoid score) of every token; with
        routing "softmax_top" the largest logits (plus bias) and the softmax over them alone."""
        T, E = logits.shape
        if routing == "softmax_top":
            z = logits.float() + (bias.float() if bias is not None else 0.0)
            best = z.topk(top, dim=-1)
            return best.indices.to(torch.int32), torch.softmax(best.values, dim=-1)
        if routing == "softmax_choice":
            s = torch.softmax(logits.float(), dim=-1)
            choice = s + (bias.float() if bias is not None else 0.0)
            per = E // group_count
            grouped = choice.view(T, group_count, per)
            kept = grouped.max(-1).values.topk(group_keep, dim=-1).indices
            allowed = torch.zeros((T, group_count), dtype=torch.bool, device=logits.device)
            allowed.scatter_(1, kept, True)
            masked = grouped.masked_fill(~allowed[:, :, None], float("-inf")).view(T, E)
            ids = masked.topk(top, dim=-1).indices
            w = s.gather(1, ids)
            return ids.to(torch.int32), (w / (w.sum(-1, keepdim=True) + 1e-20)).float()
        s = torch.sigmoid(logits.float())
        per = E // group_count
        grouped = s.view(T, group_count, per)
        group_score = grouped.topk(min(2, per), dim=-1).values.sum(-1)
        kept = group_score.topk(group_keep, dim=-1).indices
        allowed = torch.zeros((T, group_count), dtype=torch.bool, device=logits.device)
        allowed.scatter_(1, kept, True)
        masked = grouped.masked_fill(~allowed[:, :, None], float("-inf")).view(T, E)
        ids = masked.topk(top, dim=-1).indices
        return ids.to(torch.int32), (s.gather(1, ids) * scale).float()

    def moe_experts(self, x, ids, weights, up, down, num_experts, act="relu2", add=None, gated=False, add_gate=None):
        """sum over a token's experts e of weight * act(x Wu_e^T) Wd_e^T (+ add); up [E * ff, K], down [E * K, ff].
        gated: up [E * 2 ff, K] holds an expert's gate rows, then its up rows, and the hidden layer is
        act(x Wg_e^T) * (x Wu_e^T)."""
        T, K = x.shape
        ff = up.shape[0] // num_experts // (2 if gated else 1)
        out = torch.zeros((T, K), dtype=torch.float32, device=x.device)
        for e in range(num_experts):
            hit = ids == e
            rows = hit.any(-1)
            if bool(rows.any()) and gated:
                both = x[rows].float() @ up[2 * e * ff:2 * (e + 1) * ff].float().T
                h = (self._activation(both[:, :ff], act) * both[:, ff:]).to(x.dtype).float()
                y = (h @ down[e * K:(e + 1) * K].float().T).to(x.dtype).float()
                out[rows] += (weights * hit)[rows].sum(-1, keepdim=True) * y
            elif bool(rows.any()):
                h = self._activation((x[rows].float() @ up[e * ff:(e + 1) * ff].float().T), act).to(x.dtype).float()
                y = (h @ down[e * K:(e + 1) * K].float().T).to(x.dtype).float()
                out[rows] += (weights * hit)[rows].sum(-1, keepdim=True) * y
        identity = ids >= num_experts               # such a choice gives the token's input back
        if bool(identity.any()):
            out += (weights * identity).sum(-1, keepdim=True) * x.float()
        if add is not None:
            out += add.float() * (torch.sigmoid(add_gate.float())[:, None] if add_gate is not None else 1.0)
        return out.to(x.dtype)

    # feed-forward (activation.py:8-11)
    def act_mul(self, gate_up, act="silu", out=None):
        inner = gate_up.shape[1] // 2
        g, u = gate_up[:, :inner].float(), gate_up[:, inner:].float()
        if act == "silu":
            a = g * torch.sigmoid(g)
        elif act == "relu":
            a = torch.relu(g)
        elif act == "gelu_tanh":
            a = 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
        else:
            raise ValueError(act)
        y = (a * u).to(gate_up.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def silu_mul(self, gate_up, out=None):
        return self.act_mul(gate_up, "silu", out)

    def linear_act_mul(self, x, weight, act="silu"):
        return self.act_mul(self.linear(x, weight), act)

    def linear(self, x, weight, bias=None, out_float32=False, out=None, deferred=False):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        y = y if out_float32 else y.to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear_silu_mul(self, x, weight):
        return self.silu_mul(self.linear(x, weight))

    # position encoding (rotary_embedding.py:29-35)
    def rotary_table(self, inv_freq, num_positions):
        t = torch.arange(num_positions, dtype=torch.float32, device=inv_freq.device)
        ang = t[:, None] * inv_freq[None, :]
        return torch.cat((ang.cos(), ang.sin()), dim=-1)

    def qk_norm_rope_store(self, qkv, num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps, table,
                           positions, slots, k_cache, v_cache, max_position=None):
        if table is not None:
            assert max_position is not None and max_position <= table.shape[0], "a position has no row in the table"
        T = qkv.shape[0]
        D = head_dim
        qd, kd = num_heads * D, num_kv_heads * D
        dt = qkv.dtype

        def prepare(x, heads, w):
            x = x.float().reshape(T, heads, D)
            if w is not None:
                x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
                x = _round(_round(x, dt) * w.float(), dt)
            if table is not None:
                row = table[positions.long()]                       # [T, R]: the first R channels of a head are rotated
                R = row.shape[1]
                cos, sin = row[:, None, : R // 2], row[:, None, R // 2:]
                x1, x2 = x[..., : R // 2], x[..., R // 2:R]
                x = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., R:]), dim=-1)
            return x.to(dt)

        q = prepare(qkv[:, :qd], num_heads, q_weight)
        qkv[:, :qd] = q.reshape(T, qd)
        if num_kv_heads:
            k = prepare(qkv[:, qd:qd + kd], num_kv_heads, k_weight)
            qkv[:, qd:qd + kd] = k.reshape(T, kd)
            if k_cache is not None:
                page_size = k_cache.shape[2]
                v = qkv[:, qd + kd:].reshape(T, num_kv_heads, D)
                s = slots.long()
                ok = s >= 0
                page, off = s[ok] // page_size, s[ok] % page_size
                vt = v_cache.shape[4]
                k_cache[page, :, off, :] = k[ok]
                v_cache[page, :, off // vt, :, off % vt] = v[ok]
        return qkv[:, :qd]

    def rotary_step_table(self, inv_freq, positions):
        ang = positions.float()[:, None] * inv_freq[None, :]
        return torch.cat((ang.cos(), ang.sin()), dim=-1)

    def qk_rownorm_store(self, qkv, num_heads, num_kv_heads, head_dim, v_head_dim, q_weight, k_weight, eps,
                         positions, temp_coef, temp_every, slots, k_cache, v_cache, rot_table=None, norm_per_head=False,
                         rot_interleaved=False, v_norm=False, v_first_in=None, v_mix=None, v_first_out=None):
        """q and k normed over the whole projection, q times its position's temperature, both rotated by
        the rows of rot_table (one per token: cosines, then sines, for the first channels of a head),
        k and v stored."""
        T = qkv.shape[0]
        qd, kd = num_heads * head_dim, num_kv_heads * head_dim
        dt = qkv.dtype

        def turn(x, heads):
            if rot_table is None:
                return x
            R = rot_table.shape[1]
            x = x.reshape(T, heads, head_dim)
            cos, sin = rot_table[:, None, : R // 2], rot_table[:, None, R // 2:]
            if rot_interleaved:
                a, b = x[..., 0:R:2], x[..., 1:R:2]
                pairs = torch.stack((a * cos - b * sin, b * cos + a * sin), dim=-1).reshape(T, heads, R)
                return torch.cat((pairs, x[..., R:]), dim=-1).reshape(T, heads * head_dim)
            a, b = x[..., : R // 2], x[..., R // 2:R]
            return torch.cat((a * cos - b * sin, b * cos + a * sin, x[..., R:]), dim=-1).reshape(T, heads * head_dim)
        def normed(x, heads, w):
            if norm_per_head:               # every head by itself, with a weight of the head's size
                x = x.reshape(T, heads, head_dim)
                return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).reshape(T, heads * head_dim)
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        q = qkv[:, :qd].float()
        if q_weight is not None:
            q = normed(q, num_heads, q_weight)
        if temp_coef:
            steps = torch.div(positions.long() + 1, int(temp_every), rounding_mode="floor").float()
            q = q * (1.0 + temp_coef * torch.log(steps + 1.0))[:, None]
        qkv[:, :qd] = turn(q, num_heads).to(dt)
        if num_kv_heads:
            k = qkv[:, qd:qd + kd].float()
            if k_weight is not None:
                k = normed(k, num_kv_heads, k_weight)
            qkv[:, qd:qd + kd] = turn(k, num_kv_heads).to(dt)
            v = qkv[:, qd + kd:].float()
            if v_norm:
                v = v.reshape(T, num_kv_heads, v_head_dim)
                v = (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, num_kv_heads * v_head_dim)
            if v_first_out is not None:
                v_first_out.copy_(v)
            if v_first_in is not None:
                v = (1.0 - v_mix.float()) * v + v_mix.float() * v_first_in
            qkv[:, qd + kd:] = v.to(dt)
            if k_cache is not None:
                page_size, vt = k_cache.shape[2], v_cache.shape[4]
                s = slots.long()
                ok = s >= 0
                page, off = s[ok] // page_size, s[ok] % page_size
                k_cache[page, :, off, :] = qkv[:, qd:qd + kd].reshape(T, num_kv_heads, head_dim)[ok]
                v_cache[page, :, off // vt, :, off % vt] = qkv[:, qd + kd:].reshape(T, num_kv_heads, v_head_dim)[ok]
        return qkv[:, :qd]

    def sigmoid_mul(self, x, gate, out=None):
        """x * sigmoid(gate), entry by entry; in place unless out is given."""
        y = (x.float() * torch.sigmoid(gate.float())).to(x.dtype)
        out = x if out is None else out
        out.copy_(y)
        return out

    def channel_delta(self, proj, decay_in, gate_in, heads, kv_heads, dim, vdim, taps, conv_w, dt_bias, a_log, norm_w,
                      eps, conv_state, s_state, batch, out=None):
        """Token by token: the three convolutions over the request's last inputs, unit-norm q and k, beta, the
        decay per key channel, S <- diag(a) S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q, then the norm per
        head and the gate."""
        T = proj.shape[0]
        qk, vv = kv_heads * dim, heads * vdim
        C = 2 * qk + vv
        p = proj.float()
        raw, beta = p[:, :C], torch.sigmoid(p[:, C:C + heads])
        step = torch.nn.functional.softplus(decay_in.float() + dt_bias.float(), threshold=1e9).reshape(T, heads, dim)
        decay = torch.exp(-torch.exp(a_log.float())[None, :, None] * step)
        o = torch.zeros((T, heads, vdim), dtype=torch.float32, device=proj.device)
        per = heads // kv_heads
        slots = batch.state_slots.tolist()
        t = 0
        for s, (start, n) in enumerate(zip(batch.starts, batch.q_lens)):
            slot = slots[s]
            hist = conv_state[slot].clone() if start > 0 else torch.zeros_like(conv_state[slot])      # [C, taps - 1]
            S = s_state[slot].clone() if start > 0 else torch.zeros_like(s_state[slot])               # [heads, dim, vdim]
            for i in range(t, t + n):
                window = torch.cat((hist, raw[i][:, None]), dim=1)                                    # [C, taps]
                c = (window * conv_w.float()).sum(-1)
                c = c * torch.sigmoid(c)
                hist = window[:, 1:]
                q = c[:qk].reshape(kv_heads, dim)
                k = c[qk:2 * qk].reshape(kv_heads, dim)
                v = c[2 * qk:].reshape(heads, vdim)
                q = (q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5).repeat_interleave(per, 0)
                k = (k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(per, 0)
                S = decay[i][:, :, None] * S
                u = beta[i][:, None] * (v - torch.einsum("hdv,hd->hv", S, k))
                S = S + k[:, :, None] * u[:, None, :]
                o[i] = torch.einsum("hdv,hd->hv", S, q)
            conv_state[slot] = hist
            s_state[slot] = S
            t += n
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
        y = (o.reshape(T, vv) * torch.sigmoid(gate_in.float())).to(proj.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    RETENTION_CHUNK = 4

    def retention(self, proj, heads, dim, v_dim, state, decay_powers, inv_freq, k_scale, eps, batch, out=None):
        """Token by token: S <- decay S + k v^T, o = S^T q, then o / rms(o) * silu(g) per head."""
        T = proj.shape[0]
        qk, vv = heads * dim, heads * v_dim
        p = proj.float()
        q, k = p[:, :qk].reshape(T, heads, dim), p[:, qk:2 * qk].reshape(T, heads, dim)
        v, g = p[:, 2 * qk:2 * qk + vv].reshape(T, heads, v_dim), p[:, 2 * qk + vv:]
        pos = torch.cat([torch.arange(s, s + n) for s, n in zip(batch.starts, batch.q_lens)]).to(proj.device)
        if inv_freq is not None:
            half = inv_freq.shape[0]
            ang = pos.float()[:, None] * inv_freq[None, :]
            cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]

            def turn(x):
                a, b = x[..., :half], x[..., half:2 * half]
                return torch.cat((a * cos - b * sin, b * cos + a * sin, x[..., 2 * half:]), dim=-1)
            q, k = turn(q), turn(k)
        k = k * k_scale
        decay = decay_powers[:, 1].float()
        o = torch.zeros((T, heads, v_dim), dtype=torch.float32, device=proj.device)
        t = 0
        slots = batch.state_slots.tolist()
        for s, (start, n) in enumerate(zip(batch.starts, batch.q_lens)):
            S = state[slots[s]].clone() if start > 0 else torch.zeros_like(state[slots[s]])
            for i in range(t, t + n):
                S = decay[:, None, None] * S + k[i][:, :, None] * v[i][:, None, :]
                o[i] = torch.einsum("hdv,hd->hv", S, q[i])
            state[slots[s]] = S
            t += n
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        y = (o.reshape(T, vv) * (g * torch.sigmoid(g))).to(proj.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def state_space(self, proj, heads, vdim, n_state, groups, taps, conv_w, conv_b, dt_bias, a_log, d_skip, norm_w,
                    norm_groups, eps, conv_state, ssm_state, batch, out=None):
        """Token by token: the convolution over the request's last inputs, the step size, the state's
        decay and update, the read-out, the gate and the grouped norm."""
        T = proj.shape[0]
        inner, gn = heads * vdim, groups * n_state
        C = inner + 2 * gn
        p = proj.float()
        z, xbc, dt_raw = p[:, :inner], p[:, inner:inner + C], p[:, inner + C:]
        y = torch.zeros((T, inner), dtype=torch.float32, device=proj.device)
        slots = batch.state_slots.tolist()
        a = -torch.exp(a_log.float())
        per = heads // groups
        t = 0
        for s, (start, n) in enumerate(zip(batch.starts, batch.q_lens)):
            slot = slots[s]
            hist = conv_state[slot].clone() if start > 0 else torch.zeros_like(conv_state[slot])      # [C, taps - 1]
            S = ssm_state[slot].clone() if start > 0 else torch.zeros_like(ssm_state[slot])           # [heads, N, P]
            for i in range(t, t + n):
                window = torch.cat((hist, xbc[i][:, None]), dim=1)                                    # [C, taps]
                c = (window * conv_w.float()).sum(-1) + conv_b.float()
                c = (c * torch.sigmoid(c)).to(proj.dtype).float()
                hist = window[:, 1:]
                x = c[:inner].reshape(heads, vdim)
                B = c[inner:inner + gn].reshape(groups, n_state).repeat_interleave(per, 0)
                Cc = c[inner + gn:].reshape(groups, n_state).repeat_interleave(per, 0)
                dt = torch.nn.functional.softplus(dt_raw[i] + dt_bias.float(), threshold=1e9)
                S = torch.exp(a * dt)[:, None, None] * S + dt[:, None, None] * B[:, :, None] * x[:, None, :]
                y[i] = (torch.einsum("hnp,hn->hp", S, Cc) + d_skip.float()[:, None] * x).reshape(inner)
            conv_state[slot] = hist
            ssm_state[slot] = S
            t += n
        y = y * (z * torch.sigmoid(z))
        y = y.reshape(T, norm_groups, inner // norm_groups)
        y = (y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, inner) * norm_w.float()
        y = y.to(proj.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    # attention (attention.py:64-75): token by token through the block table
    def paged_attention(self, q, num_heads, num_kv_heads, head_dim, k_cache, v_cache, batch, group, scale,
                        window=None, out=None, v_head_dim=None, sinks=None, chunk=None, softcap=None, keep_first=0,
                        sigmoid_bias=None):
        T = q.shape[0]
        D, G = head_dim, num_heads // num_kv_heads
        DV = v_head_dim or head_dim
        page_size = k_cache.shape[2]
        tables = batch.groups[group].block_tables
        o = torch.zeros((T, num_heads * DV), dtype=torch.float32, device=q.device)
        pos_l, seq_l = batch.positions.tolist(), batch.token_seq.tolist()
        for t in range(T):
            pos, seq = pos_l[t], seq_l[t]
            first = max(0, pos - window + 1) if window else 0
            if chunk:
                first = max(first, pos // chunk * chunk)
            js = torch.arange(first, pos + 1, device=q.device)
            if window and keep_first and first > 0:       # the sequence's first positions stay in sight
                js = torch.cat((torch.arange(0, min(keep_first, first), device=q.device), js))
            pages = tables[seq].long()[js // page_size]
            assert bool((pages >= 0).all()), "a visible key has no page"
            offs = js % page_size
            keys = k_cache[pages, :, offs, :].float()                # [n, Hkv, D]
            vt = v_cache.shape[4]
            vals = v_cache[pages, :, offs // vt, :, offs % vt].float()   # [n, Hkv, D]
            qt = q[t].float().reshape(num_heads, D)
            for h in range(num_heads):
                s = (keys[:, h // G] @ qt[h]) * scale
                if softcap:
                    s = softcap * torch.tanh(s / softcap)
                if sigmoid_bias is not None:   # every key by itself, no normalisation
                    p = torch.sigmoid(s + sigmoid_bias[h].float())
                elif sinks is not None:       # one more term in the denominator: a key without a value
                    p = torch.softmax(torch.cat((s, sinks[h:h + 1].float())), dim=0)[:-1]
                else:
                    p = torch.softmax(s, dim=0)
                o[t, h * DV:(h + 1) * DV] = p @ vals[:, h // G]
        y = o.to(q.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    # attention through a latent
    def latent_prepare(self, proj, heads, dim, rot, rank, weight, eps, rot_table, slots, k_cache, v_cache):
        T = proj.shape[0]
        dt = proj.dtype
        qd = heads * (dim + rot)
        cos, sin = rot_table[:, : rot // 2], rot_table[:, rot // 2:]

        def turn(x):                                    # [..., rot] with the tokens first
            a, b = x[..., 0::2], x[..., 1::2]
            c, s = (cos, sin) if x.dim() == 2 else (cos[:, None], sin[:, None])
            return torch.stack((a * c - b * s, b * c + a * s), dim=-1).reshape(x.shape)
        q = proj[:, :qd].float().reshape(T, heads, dim + rot)
        q2 = torch.zeros((T, heads, rank + rot), dtype=dt, device=proj.device)
        q2[:, :, rank:] = turn(q[:, :, dim:]).to(dt)
        if k_cache is not None:
            c = proj[:, qd:qd + rank].float()
            c = (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(dt)
            kr = turn(proj[:, qd + rank:].float()).to(dt)
            page_size, vt = k_cache.shape[2], v_cache.shape[4]
            s = slots.long()
            ok = s >= 0
            page, off = s[ok] // page_size, s[ok] % page_size
            k_cache[page, 0, off, :] = torch.cat((c, kr), dim=-1)[ok]
            v_cache[page, 0, off // vt, :, off % vt] = c[ok]
        return q2.reshape(T, heads * (rank + rot))

    def latent_attention(self, q2, heads, rank, rot, k_cache, v_cache, batch, group, scale, sinks=None):
        return self.paged_attention(q2, heads, 1, rank + rot, k_cache, v_cache, batch, group, scale, None, v_head_dim=rank,
                                    sinks=sinks)

    def heads_linear(self, x, x_head, w, heads, n_out, k_in, transposed, y, y_head, y_offset=0):
        wh = w.float().reshape(heads, k_in, n_out).transpose(1, 2) if transposed else w.float().reshape(heads, n_out, k_in)
        for h in range(heads):
            xh = x[:, h * x_head: h * x_head + k_in].float()
            y[:, h * y_head + y_offset: h * y_head + y_offset + n_out] = (xh @ wh[h].T).to(y.dtype)
        return y

    # sampling (sampler.py:8-12), same counter-based noise as the kernel
    def sample(self, logits, temperatures, keys):
        import math
        M = (1 << 64) - 1

        def mix(z):
            z = (z + 0x9E3779B97F4A7C15) & M
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
            return z ^ (z >> 31)

        out = []
        for r in range(logits.shape[0]):
            l = logits[r].double().cpu()
            t = float(temperatures[r])
            if t > 0:
                key = int(keys[r]) & M
                noise = torch.tensor([math.log(-math.log((((mix(key ^ i)) >> 40) + 0.5) / 16777216.0))
                                      for i in range(l.numel())], dtype=torch.float64)
                l = l / t - noise
            out.append(int(torch.argmax(l)))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
