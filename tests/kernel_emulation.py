"""A plain emulation of every kernel's contract, in ordinary torch arithmetic.

It has two uses.  On a machine without a GPU it stands in for the kernel library
so that the engine's bookkeeping (cache, batching, scheduling) can be compared
with the plain implementation.  On the GPU it is each kernel's reference: the
`-m gpu` tests run a kernel and its emulation on the same operands.  It follows
the contracts written in `wllm_amd/kernels/ops.py`, not the kernels' code, and
computes in float64 when `precise` is set.
"""
from __future__ import annotations

import math

import torch


class EmulatedKernels:
    def __init__(self, precise: bool = False, splits: int = 1):
        self.acc = torch.float64 if precise else torch.float32
        self.calls = {}
        self.splits = splits        # into how many partial sums `linear` is asked to split

    def _count(self, name):
        self.calls[name] = self.calls.get(name, 0) + 1

    def run_registered(self, op, args, kwargs):
        """An operation that went through `ops.register_op`: the framework's own have their emulation
        here under their name; one that a part registered brings its own."""
        own = getattr(self, op.name, None)
        if own is not None:
            own(*args, **kwargs)
            return
        self._count(op.name)
        if op.emulate is None:
            raise NotImplementedError(f"operation {op.name!r} was registered without an emulation")
        op.emulate(*args, **kwargs)

    def embed_lookup(self, ids, table, scale, out):
        self._count("embed_lookup")
        out.copy_((table[ids.long()].to(self.acc) * scale).to(out.dtype))

    def feed_tokens(self, ids, dst, src, source):
        self._count("feed_tokens")
        for d, s in zip(dst.tolist(), src.tolist()):
            if 0 <= d < ids.shape[0] and 0 <= s < source.shape[0]:
                ids[d] = source[s]

    def rms_norm(self, x, weight, eps, offset, out, delta, rows, delta_bias=None):
        self._count("rms_norm")
        if delta is not None and delta.dim() == 3:
            total = delta[0].to(torch.float32)
            for p in range(1, delta.shape[0]):
                total = total + delta[p]
            delta = total
        if delta_bias is not None:      # a row that comes with the pending contribution
            delta = delta_bias.expand_as(x) if delta is None else delta.to(torch.float32) + delta_bias
        if rows is None:
            v = x.to(self.acc)
            if delta is not None:
                v = v + delta.to(self.acc)
                x.copy_(v.to(x.dtype))
                v = x.to(self.acc)  # the kernel normalises what it wrote back
        else:
            idx = rows.long()
            v = x[idx].to(self.acc)
            if delta is not None:
                v = (v + delta[idx].to(self.acc)).to(x.dtype).to(self.acc)
        var = v.pow(2).mean(-1, keepdim=True)
        y = v * torch.rsqrt(var + eps) * (offset + weight.to(self.acc))
        out.copy_(y.to(out.dtype))

    fused_qkv = True        # whether the emulation offers the fused projection and rotation
    fused_residual = True   # and the product that adds into the residual stream

    def linear_residual_takes(self, rows, dtype, out_features, in_features):
        return self.fused_residual and rows <= 16 and out_features % 16 == 0

    def linear_residual(self, x, weight, tiles, residual, sumsq):
        self._count("linear_residual")
        self._same_numbers(weight, tiles, 1)
        new = residual.to(self.acc) + x.to(self.acc) @ weight.to(self.acc).T
        residual.copy_(new.to(torch.float32))
        sumsq.copy_((residual.to(self.acc) ** 2).view(residual.shape[0], -1, 16).sum(-1).to(torch.float32))

    def qkv_rope_takes(self, rows, dtype, in_features, head_dim, rotary_dim):
        return self.fused_qkv and rotary_dim == head_dim and rows <= 32

    def qkv_rope(self, x, weight, tiles, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                 head_dim, page_size):
        self._count("qkv_rope")
        self._same_numbers(weight, tiles, 1)
        # the kernel rotates the float32 sums, not their rounding to the activation dtype: hand them
        # on as a stack of one partial sum
        pre = (x.to(self.acc) @ weight.to(self.acc).T).to(torch.float32)[None]
        self.rope_and_cache_write(qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads, head_dim,
                                  head_dim if inv_freq is not None else 0, page_size, parts=pre)
        self.calls["rope_and_cache_write"] -= 1

    def rope_and_cache_write(self, qkv, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads,
                             head_dim, rotary_dim, page_size, parts=None):
        self._count("rope_and_cache_write")
        n = qkv.shape[0]
        heads = num_heads + 2 * num_kv_heads
        if parts is not None:
            total = parts[0]
            for p in range(1, parts.shape[0]):
                total = total + parts[p]
            v = total.to(self.acc)
        else:
            v = qkv.to(self.acc)
        if bias is not None:
            v = v + bias.to(self.acc)
        v = v.view(n, heads, head_dim).clone()
        if inv_freq is not None:
            half = rotary_dim // 2
            ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]          # float32 angles
            cos, sin = ang.cos().to(self.acc)[:, None, :], ang.sin().to(self.acc)[:, None, :]
            r = num_heads + num_kv_heads                                              # queries and keys
            x1 = v[:, :r, :half].clone()
            x2 = v[:, :r, half:rotary_dim].clone()
            v[:, :r, :half] = x1 * cos - x2 * sin
            v[:, :r, half:rotary_dim] = x2 * cos + x1 * sin
        qkv.copy_(v.view(n, -1).to(qkv.dtype))
        if cache is not None:
            rows = qkv.view(n, heads, head_dim)
            page = (slots // page_size).long()
            off = (slots % page_size).long()
            k = rows[:, num_heads:num_heads + num_kv_heads]                           # [n, nkv, d]
            val = rows[:, num_heads + num_kv_heads:]
            kview = cache[:, 0].view(cache.shape[0], num_kv_heads, page_size, head_dim)
            vview = cache[:, 1].view(cache.shape[0], num_kv_heads, head_dim, page_size)
            kview[page, :, off, :] = k
            vview[page, :, :, off] = val

    def paged_attention(self, qkv, cache, block_tables, token_segment, seg_q_start, seg_q_len, seg_ctx_len, out,
                        num_heads, num_kv_heads, head_dim, page_size, scale, window, max_q_len, max_ctx_len,
                        plan=None, softcap=0.0, exact_weights=False, chunk=0, sinks=None):
        self._count("paged_attention")
        n = qkv.shape[0]
        n_rep = num_heads // num_kv_heads
        q_all = qkv[:, :num_heads * head_dim].reshape(n, num_heads, head_dim).to(self.acc)
        pages = cache.shape[0]
        kview = cache[:, 0].view(pages, num_kv_heads, page_size, head_dim)
        vview = cache[:, 1].view(pages, num_kv_heads, head_dim, page_size)
        for s in range(block_tables.shape[0]):
            q0, ql, cl = int(seg_q_start[s]), int(seg_q_len[s]), int(seg_ctx_len[s])
            if ql == 0:
                continue
            npages = -(-cl // page_size)
            ids = block_tables[s, :npages].long()
            k = kview[ids].permute(0, 2, 1, 3).reshape(npages * page_size, num_kv_heads, head_dim)[:cl].to(self.acc)
            v = vview[ids].permute(0, 3, 1, 2).reshape(npages * page_size, num_kv_heads, head_dim)[:cl].to(self.acc)
            k = k.repeat_interleave(n_rep, dim=1)
            v = v.repeat_interleave(n_rep, dim=1)
            q = q_all[q0:q0 + ql]
            pos = torch.arange(cl - ql, cl, device=q.device)
            key = torch.arange(cl, device=q.device)
            allowed = key[None, :] <= pos[:, None]
            if window:
                allowed &= key[None, :] > pos[:, None] - window
            if chunk:
                allowed &= key[None, :] >= (pos[:, None] // chunk) * chunk
            scores = torch.einsum("qhd,khd->hqk", q, k) * scale
            if softcap:
                scores = softcap * torch.tanh(scores / softcap)
            # keys outside the window may hold NaN of pages given back: mask by selection, not by addition
            scores = torch.where(allowed[None], scores, torch.full_like(scores, float("-inf")))
            if sinks is not None:
                # one more term of the denominator: a column that is dropped after the softmax
                sink = sinks.to(self.acc)[:, None, None].expand(-1, ql, 1)
                probs = torch.softmax(torch.cat([scores, sink], dim=-1), dim=-1)[..., :-1]
            else:
                probs = torch.softmax(scores, dim=-1)
            v = torch.where(torch.isnan(v), torch.zeros_like(v), v) if (window or chunk) else v
            o = torch.einsum("hqk,khd->qhd", probs, v)
            out[q0:q0 + ql] = o.reshape(ql, num_heads * head_dim).to(out.dtype)

    def plan_paged_attention(self, *args):
        return None

    def head_prepare(self, rows, bias, positions, inv_freq, slots, cache, num_heads, num_kv_heads, head_dim, page_size,
                     interleaved, norm_eps, values_are_keys, parts, norm_dim=None, head_norm=None, rot_scale=1.0):
        self._count("head_prepare")
        n, width = rows.shape
        if parts is not None:
            total = parts[0]
            for p in range(1, parts.shape[0]):
                total = total + parts[p]
            v = total.to(self.acc)
        else:
            v = rows.to(self.acc)
        v = v.clone()
        if bias is not None:
            v[:, :bias.shape[0]] += bias.to(self.acc)       # the row's first columns have a bias
        r = num_heads + num_kv_heads
        heads = v[:, :r * head_dim].reshape(n, r, head_dim).clone()
        as_projected = heads[:, num_heads:].clone()
        if head_norm is not None:
            w_q, w_k, pre_eps = head_norm
            heads = heads * torch.rsqrt(heads.pow(2).sum(-1, keepdim=True) / (norm_dim or head_dim) + pre_eps)
            heads[:, :num_heads] *= w_q.to(self.acc)
            heads[:, num_heads:] *= w_k.to(self.acc)
        if inv_freq is not None:
            half = inv_freq.shape[0]
            ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]          # float32 angles
            cos, sin = (ang.cos() * rot_scale).to(self.acc)[:, None, :], (ang.sin() * rot_scale).to(self.acc)[:, None, :]
            if interleaved:
                x1, x2 = heads[..., 0:2 * half:2].clone(), heads[..., 1:2 * half:2].clone()
                heads[..., 0:2 * half:2] = x1 * cos - x2 * sin
                heads[..., 1:2 * half:2] = x2 * cos + x1 * sin
            else:
                x1, x2 = heads[..., :half].clone(), heads[..., half:2 * half].clone()
                heads[..., :half] = x1 * cos - x2 * sin
                heads[..., half:2 * half] = x2 * cos + x1 * sin
        if norm_eps is not None:
            heads = heads * torch.rsqrt(heads.pow(2).sum(-1, keepdim=True) / (norm_dim or head_dim) + norm_eps)
        v[:, :r * head_dim] = heads.reshape(n, -1)
        rows.copy_(v.to(rows.dtype))
        if cache is not None:
            page = (slots // page_size).long()
            off = (slots % page_size).long()
            k = rows[:, num_heads * head_dim:r * head_dim].reshape(n, num_kv_heads, head_dim)
            if values_are_keys:
                val = as_projected.to(rows.dtype)
            else:
                val = rows[:, r * head_dim:(r + num_kv_heads) * head_dim].reshape(n, num_kv_heads, head_dim)
            kview = cache[:, 0].view(cache.shape[0], num_kv_heads, page_size, head_dim)
            vview = cache[:, 1].view(cache.shape[0], num_kv_heads, head_dim, page_size)
            kview[page, :, off, :] = k
            vview[page, :, :, off] = val

    def sigmoid_gate(self, a, gate, out, per=1):
        self._count("sigmoid_gate")
        g = torch.sigmoid(gate.to(self.acc)).repeat_interleave(per, dim=1)
        out.copy_((a.to(self.acc) * g).to(out.dtype))

    # ---- the general norm step, the band norm, the token input's lookup, the product head by head ----
    def _normed(self, v, recipe):
        if recipe is None:
            return v
        if recipe.kind == "layer":
            v = v - v.mean(-1, keepdim=True)
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + recipe.eps) * (recipe.offset + recipe.weight.to(self.acc))

    def norm_add(self, x, delta, delta_norm, out, out_norm, rows, conv=None):
        self._count("norm_add")
        idx = rows.long() if rows is not None else slice(None)
        v = x[idx].to(self.acc)
        if delta is not None:
            if delta.dim() == 3:
                total = delta[0]
                for p in range(1, delta.shape[0]):
                    total = total + delta[p]
                delta = total
            v = (v + self._normed(delta[idx].to(self.acc), delta_norm)).to(x.dtype)
            if rows is None:
                x.copy_(v)
            v = v.to(self.acc)
        if conv is not None:
            weight, state, offset, slots = conv
            taps, c = weight.shape
            for r in range(x.shape[0]):
                carried = state[int(slots[r]), offset:offset + (taps - 1) * c].view(taps - 1, c)
                seq = torch.cat([carried.to(self.acc), v[r:r + 1]], dim=0)
                out[r] = (v[r] + (seq * weight.to(self.acc)).sum(0)).to(out.dtype)
                if taps > 1:
                    carried.copy_(seq[1:].float())
            return
        if out is not None:
            out.copy_(self._normed(v, out_norm).to(out.dtype))

    def band_norm(self, bands, eps):
        self._count("band_norm")
        for band in bands:
            src, weight, count, out = band[:4]
            bias = band[4] if len(band) > 4 else None
            v = src.to(self.acc)
            if bias is not None:
                v = v + bias.to(self.acc)
            y = v * torch.rsqrt(v.pow(2).sum(-1, keepdim=True) / count + eps) * weight.to(self.acc)
            cols = src.shape[1]
            result = torch.zeros(out.shape, dtype=out.dtype, device=out.device)
            result[:, :cols] = y.to(out.dtype)
            out.copy_(result)

    def gated_lookup(self, gate, ids, table, col0, out, activation):
        self._count("gated_lookup")
        z = gate.to(self.acc)
        if activation == "gelu_tanh":
            a = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
        else:
            a = z * torch.sigmoid(z)
        out.copy_((a * table[ids.long(), col0:col0 + gate.shape[1]].to(self.acc)).to(out.dtype))

    def head_linear(self, x, w, y):
        self._count("head_linear")
        heads, o, k = w.shape
        n = x.shape[0]
        r = torch.einsum("nhk,hok->nho", x.reshape(n, heads, k).to(self.acc), w.to(self.acc))
        y.copy_(r.reshape(n, heads * o).to(y.dtype))

    # ---- the state-space mixer's three kernels ----
    def causal_conv(self, inp, weight, bias, state, carried_offset, token_segment, seg_q_start, seg_q_len, state_slots, out):
        self._count("causal_conv")
        c, taps = weight.shape
        for s in range(seg_q_start.shape[0]):
            q0, ql, slot = int(seg_q_start[s]), int(seg_q_len[s]), int(state_slots[s])
            if ql == 0:
                continue
            carried = state[slot, carried_offset:carried_offset + (taps - 1) * c].view(taps - 1, c)
            seq = torch.cat([carried.to(self.acc), inp[q0:q0 + ql].to(self.acc)], dim=0)
            acc = bias.to(self.acc).expand(ql, -1).clone()
            for k in range(taps):
                acc = acc + seq[k:k + ql] * weight[:, k].to(self.acc)
            out[q0:q0 + ql] = (acc * torch.sigmoid(acc)).to(out.dtype)
            if taps > 1:
                carried.copy_(seq[ql:].to(torch.float32))

    def stream_conv(self, x, weight, state, carried_offset, token_segment, seg_q_start, seg_q_len, state_slots, out,
                    single_tokens=False):
        self._count("stream_conv")
        assert not single_tokens or all(int(n) == 1 for n in seg_q_len)
        taps, c = weight.shape
        for s in range(seg_q_start.shape[0]):
            q0, ql, slot = int(seg_q_start[s]), int(seg_q_len[s]), int(state_slots[s])
            if ql == 0:
                continue
            carried = state[slot, carried_offset:carried_offset + (taps - 1) * c].view(taps - 1, c)
            seq = torch.cat([carried.to(self.acc), x[q0:q0 + ql].to(self.acc)], dim=0)
            acc = x[q0:q0 + ql].to(self.acc).clone()
            for k in range(taps):
                acc = acc + seq[k:k + ql] * weight[k].to(self.acc)
            out[q0:q0 + ql] = acc.to(out.dtype)
            if taps > 1:
                carried.copy_(seq[ql:ql + taps - 1].float())

    def ssm_scan(self, xbc, dt, dt_bias, a_log, d_skip, state, seg_q_start, seg_q_len, state_slots, y, heads, groups,
                 state_size, head_dim, steps=None):
        self._count("ssm_scan")
        inner, n_s = heads * head_dim, state_size
        per = heads // groups
        a = -torch.exp(a_log.to(self.acc))
        for s in range(seg_q_start.shape[0]):
            q0, ql, slot = int(seg_q_start[s]), int(seg_q_len[s]), int(state_slots[s])
            if ql == 0:
                continue
            S = state[slot, :heads * n_s * head_dim].view(heads, n_s, head_dim)
            cur = S.to(self.acc)
            for t in range(q0, q0 + ql):
                x = xbc[t, :inner].to(self.acc).view(heads, head_dim)
                b = xbc[t, inner:inner + groups * n_s].to(self.acc).view(groups, n_s).repeat_interleave(per, dim=0)
                c = xbc[t, inner + groups * n_s:].to(self.acc).view(groups, n_s).repeat_interleave(per, dim=0)
                step = torch.nn.functional.softplus(dt[t].to(self.acc) + dt_bias.to(self.acc), threshold=1e9)
                cur = torch.exp(a * step)[:, None, None] * cur + step[:, None, None] * b[:, :, None] * x[:, None, :]
                cur = cur.to(torch.float32).to(self.acc)        # the state lives in float32
                yt = torch.einsum("hnp,hn->hp", cur, c) + d_skip.to(self.acc)[:, None] * x
                y[t] = yt.reshape(inner).to(y.dtype)
            S.copy_(cur.to(torch.float32))

    def gated_group_norm(self, y, z, weight, out, groups, eps):
        self._count("gated_group_norm")
        n, w = y.shape
        zz = z.to(self.acc)
        v = (y.to(self.acc) * zz * torch.sigmoid(zz)).view(n, groups, w // groups)
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        out.copy_((v.reshape(n, w) * weight.to(self.acc)).to(out.dtype))

    def copy_columns(self, src, out, scale=1.0):
        self._count("copy_columns")
        out.copy_(src if scale == 1.0 else (src.to(self.acc) * scale).to(out.dtype))

    # ---- a matrix memory a head -------------------------------------------------------------------
    def memory_inputs(self, row, positions, inv_freq, qk, heads, head_dim, q_scale, k_scale):
        self._count("memory_inputs")
        n, width = row.shape[0], heads * head_dim
        v = row[:, :2 * width].to(self.acc).reshape(n, 2 * heads, head_dim).clone()
        if inv_freq is not None:
            half = inv_freq.shape[0]
            ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]          # float32 angles
            cos, sin = ang.cos().to(self.acc)[:, None, :], ang.sin().to(self.acc)[:, None, :]
            a, b = v[..., :half].clone(), v[..., half:2 * half].clone()
            v[..., :half] = a * cos - b * sin
            v[..., half:2 * half] = b * cos + a * sin
        v = v.reshape(n, 2, width)
        qk[0].copy_((v[:, 0] * q_scale).to(torch.float32))
        qk[1].copy_((v[:, 1] * k_scale).to(torch.float32))

    def memory_forget_inputs(self, row, bias, lower, qkf, width, q_activation):
        self._count("memory_forget_inputs")
        acc = self.acc
        q, z = row[:, :width].to(acc), row[:, width:2 * width].to(acc)
        if bias is not None:
            z = z + bias.to(acc)
        low = lower.to(acc) if lower is not None else torch.zeros(width, dtype=acc)
        f = low + (1.0 - low) * torch.sigmoid(z)
        qkf[0].copy_((q * torch.sigmoid(q) if q_activation == "silu" else q).float())
        qkf[1].copy_((1.0 - f).float())
        qkf[2].copy_(f.float())

    def memory_gates(self, gates, i_bias, f_bias, state, m_offset, seg_q_start, seg_q_len, state_slots, steps, heads, cap):
        self._count("memory_gates")
        acc = self.acc
        z = gates.to(acc)
        zi, zf = z[:, :heads], z[:, heads:2 * heads]
        if i_bias is not None:
            zi = zi + i_bias.to(acc)
        if f_bias is not None:
            zf = zf + f_bias.to(acc)
        if cap:
            zi, zf = cap * torch.tanh(zi / cap), cap * torch.tanh(zf / cap)
        log_i, log_f = zi, torch.nn.functional.logsigmoid(zf)
        for seg in range(seg_q_start.shape[0]):
            start, length, slot = int(seg_q_start[seg]), int(seg_q_len[seg]), int(state_slots[seg])
            m = state[slot, m_offset:m_offset + heads].to(acc).clone()
            for t in range(start, start + length):
                m_new = torch.maximum(log_f[t] + m, log_i[t])
                steps[0, t] = torch.exp(log_f[t] + m - m_new).float()
                steps[1, t] = torch.exp(log_i[t] - m_new).float()
                steps[2, t] = torch.exp(-m_new).float()
                m = m_new
            state[slot, m_offset:m_offset + heads] = m.float()

    def memory_scan(self, qk, v, steps, decays, state, seg_q_start, seg_q_len, state_slots, y, heads, head_dim, value_dim,
                    nq=None, n_offset=0, row_decays=False):
        self._count("memory_scan")
        acc = self.acc
        size, width = heads * head_dim * value_dim, heads * head_dim
        for seg in range(seg_q_start.shape[0]):
            start, length, slot = int(seg_q_start[seg]), int(seg_q_len[seg]), int(state_slots[seg])
            S = state[slot, :size].to(acc).view(heads, head_dim, value_dim).clone()
            nv = state[slot, n_offset:n_offset + width].to(acc).view(heads, head_dim).clone() if steps is not None else None
            for t in range(start, start + length):
                q, k = qk[0, t].to(acc).view(heads, head_dim), qk[1, t].to(acc).view(heads, head_dim)
                val = v[t].to(acc).view(heads, value_dim)
                if steps is not None:
                    a, b = steps[0, t].to(acc), steps[1, t].to(acc)
                    nv = a[:, None] * nv + b[:, None] * k
                    nq[t] = (nv * q).sum(-1).float()
                elif row_decays:
                    a, b = None, torch.ones(heads, dtype=acc)
                    S = qk[2, t].to(acc).view(heads, head_dim)[:, :, None] * S
                else:
                    a, b = decays.to(acc), torch.ones(heads, dtype=acc)
                S = (1.0 if a is None else a[:, None, None]) * S + (b[:, None] * k)[:, :, None] * val[:, None, :]
                y[t] = torch.einsum("hdv,hd->hv", S, q).reshape(-1).float()
            state[slot, :size] = S.reshape(-1).float()
            if steps is not None:
                state[slot, n_offset:n_offset + width] = nv.reshape(-1).float()

    def head_norm_gate(self, y, gate, weight, out, heads, eps, activation, scale, nq=None, floor=None, den_eps=0.0):
        self._count("head_norm_gate")
        n, w = y.shape
        v = y.to(self.acc).view(n, heads, w // heads)
        if nq is not None:
            v = v / (torch.maximum(nq.to(self.acc).abs(), floor.to(self.acc)) + den_eps)[:, :, None]
        v = (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)).reshape(n, w)
        if weight is not None:
            v = v * weight.to(self.acc)
        if activation != "none":
            z = gate.to(self.acc)
            v = v * (torch.sigmoid(z) if activation == "sigmoid" else z * torch.sigmoid(z))
        out.copy_((v * scale).to(out.dtype))

    # ---- a mixture of experts ---------------------------------------------------------------------
    def moe_route(self, x, router, ids, weights, groups, keep, eps, scoring="softmax", normalize=True):
        self._count("moe_route")
        n, experts, top = x.shape[0], router.shape[0], ids.shape[1]
        z = x.to(self.acc) @ router.to(self.acc).T
        s = torch.sigmoid(z) if scoring == "sigmoid" else torch.softmax(z, dim=-1)
        allowed = torch.ones(n, experts, dtype=torch.bool)
        if keep < groups:
            per = experts // groups
            best = s.view(n, groups, per).max(-1).values
            kept = torch.zeros(n, groups, dtype=torch.bool)
            for r in range(n):
                order = sorted(range(groups), key=lambda g: (-float(best[r, g]), g))
                kept[r, order[:keep]] = True
            allowed = kept[:, :, None].expand(n, groups, per).reshape(n, experts)
        for r in range(n):
            order = sorted([e for e in range(experts) if allowed[r, e]], key=lambda e: (-float(s[r, e]), e))[:top]
            chosen = s[r, order]
            ids[r] = torch.tensor(order, dtype=torch.int32)
            weights[r] = (chosen / (chosen.sum() + eps) if normalize else chosen).float()

    def moe_plan(self, ids, plan, experts, tile_rows=16):
        self._count("moe_plan")
        flat = ids.reshape(-1).tolist()
        max_tiles = len(flat) // tile_rows + experts
        plan.fill_(-7)                       # what the kernels must not read
        tiles = 0
        for e in range(experts):
            mine = [a for a, x in enumerate(flat) if x == e]
            for t0 in range(0, len(mine), tile_rows):
                rows = mine[t0:t0 + tile_rows]
                plan[1 + tiles] = e
                at = 1 + max_tiles + tile_rows * tiles
                plan[at:at + tile_rows] = torch.tensor(rows + [-1] * (tile_rows - len(rows)), dtype=torch.int32)
                tiles += 1
        plan[0] = tiles

    def _plan_rows(self, plan, experts, assignments, tile_rows=16):
        max_tiles = assignments // tile_rows + experts
        for t in range(int(plan[0])):
            at = 1 + max_tiles + tile_rows * t
            yield int(plan[1 + t]), [a for a in plan[at:at + tile_rows].tolist() if a >= 0]

    def moe_experts_up(self, x, w, plan, act, top, activation, tiles=None, tile_rows=16, in_weights=None):
        self._count("moe_experts_up")
        ff = w.shape[1] // 2
        for e, rows in self._plan_rows(plan, w.shape[0], act.shape[0], tile_rows):
            h = x[[a // top for a in rows]].to(self.acc)
            z, u = h @ w[e, :ff].to(self.acc).T, h @ w[e, ff:].to(self.acc).T
            if in_weights is not None:
                factor = in_weights.reshape(-1)[rows].to(self.acc)[:, None]
                z, u = z * factor, u * factor
            if activation == "gelu_tanh":
                z = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
            else:
                z = z * torch.sigmoid(z)
            act[rows] = (z * u).to(act.dtype)

    def moe_experts_down(self, act, w, plan, weights, out, tiles=None, tile_rows=16, weighted=True):
        self._count("moe_experts_down")
        n, top = weights.shape
        flat = weights.reshape(-1) if weighted else torch.ones(weights.numel())
        for e, rows in self._plan_rows(plan, w.shape[0], act.shape[0], tile_rows):
            y = act[rows].to(self.acc) @ w[e].to(self.acc).T
            for a, r in zip(rows, y):
                out[a % top, a // top] = (r * flat[a].to(self.acc)).float()

    def moe_experts_up_tiled(self, x, w, plan, act, top, activation, in_weights=None):
        self._count("moe_experts_up_tiled")
        self.moe_experts_up(x, w, plan, act, top, activation, tile_rows=128, in_weights=in_weights)

    def moe_experts_down_tiled(self, act, w, plan, weights, out, weighted=True):
        self._count("moe_experts_down_tiled")
        self.moe_experts_down(act, w, plan, weights, out, tile_rows=128, weighted=weighted)

    def stream_add(self, x, addend, delta, delta_bias):
        self._count("stream_add")
        v = x.to(self.acc)
        if delta is not None:
            if delta.dim() == 3:
                total = delta[0]
                for p in range(1, delta.shape[0]):
                    total = total + delta[p]
                delta = total
            v = v + delta.to(self.acc)
        if delta_bias is not None:
            v = v + delta_bias.to(self.acc)
        if addend is not None:
            v = v + addend.to(self.acc)
        x.copy_(v.to(x.dtype))

    def linear_splits(self, rows, out_features, in_features, dtype):
        return self.splits

    def tile_weight(self, weight, tiles):
        """bfloat16: [n, k] -> [band][step][g][i][8]: lane 16g + i of a wavefront holds w[16 band + i][32 step + 8g .. +8].
        float32: [n, k] -> [band][chunk][g][i][4] with rows and keys padded with zeros to multiples of 16."""
        n, k = weight.shape
        if weight.dtype == torch.float32:
            padded = torch.zeros(-(-n // 16) * 16, -(-k // 16) * 16, dtype=weight.dtype, device=weight.device)
            padded[:n, :k] = weight
            tiles.copy_(padded.view(-1, 16, padded.shape[1] // 16, 4, 4).permute(0, 2, 3, 1, 4).reshape(-1))
            return
        padded = torch.zeros(-(-n // 16) * 16, k, dtype=weight.dtype, device=weight.device)
        padded[:n] = weight
        tiles.copy_(padded.view(-1, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1))

    def _same_numbers(self, weight, tiles, halves):
        """A tile-major copy must hold the weight's numbers: the emulation computes from the weight."""
        if tiles is None:
            return
        if weight.dtype == torch.float32:
            n, k = weight.shape
            kp = -(-k // 16) * 16
            back = tiles.view(-1, kp // 16, 4, 16, 4).permute(0, 3, 1, 2, 4).reshape(-1, kp)[:n, :k]
            assert torch.equal(back, weight), "the tile-major copy differs from the weight"
            return
        n, k = weight.shape[0] // halves, weight.shape[1]
        size = -(-n // 16) * 16 * k
        for h in range(halves):
            back = tiles[h * size:(h + 1) * size].view(-1, k // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(-1, k)[:n]
            assert torch.equal(back, weight[h * n:(h + 1) * n]), "the tile-major copy differs from the weight"

    def linear(self, x, weight, out, tiles=None):
        self._count("linear")
        self._same_numbers(weight, tiles, 1)
        if out.dim() == 3:
            k = x.shape[1]
            edges = [round(i * k / out.shape[0]) for i in range(out.shape[0] + 1)]
            for p in range(out.shape[0]):
                a, b = edges[p], edges[p + 1]
                out[p].copy_((x[:, a:b].to(self.acc) @ weight[:, a:b].to(self.acc).T).to(out.dtype))
            return
        out.copy_((x.to(self.acc) @ weight.to(self.acc).T).to(out.dtype))

    fused_norm = True       # and the gated product with the norm on load

    def gated_linear_norm_takes(self, rows, dtype, in_features):
        return self.fused_norm and rows <= 16

    def gated_linear_norm(self, x, weight, out, activation, tiles=None):
        self._count("gated_linear_norm")
        self._same_numbers(weight, tiles, 2)
        r = x.residual.to(self.acc)
        # the mean square comes from the sums the producer left, not from the residual itself
        inv = torch.rsqrt(x.sumsq.to(self.acc).sum(-1, keepdim=True) / r.shape[1] + x.eps)
        h = (r * inv * (x.offset + x.weight.to(self.acc))).to(x.dtype)
        gu = (h.to(self.acc) @ weight.to(self.acc).T)
        self.gated_activation(gu, out, activation)
        self.calls["gated_activation"] -= 1

    def gated_linear(self, x, weight, out, activation, scratch, tiles=None):
        self._count("gated_linear")
        self._same_numbers(weight, tiles, 2)
        gu = (x.to(self.acc) @ weight.to(self.acc).T)
        self.gated_activation(gu, out, activation)

    def gated_activation(self, gate_up, out, activation):
        self._count("gated_activation")
        i = gate_up.shape[1] // 2
        g, u = gate_up[:, :i].to(self.acc), gate_up[:, i:].to(self.acc)
        if activation == "gelu_tanh":
            a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g.pow(3))))
        elif activation == "silu":
            a = g * torch.sigmoid(g)
        else:
            raise ValueError(activation)
        out.copy_((a * u).to(out.dtype))

    def argmax_rows(self, logits, out):
        self._count("argmax_rows")
        out.copy_(logits.argmax(dim=-1).to(torch.int32))

    def sample_rows(self, logits, params, seeds, penalty_ids, penalty_offsets, out_tokens, out_logprobs,
                    truncations=True):
        from plain.sampling_plain import philox_uniform, sample_row
        self._count("sample_rows")
        for r in range(logits.shape[0]):
            t, k, p, mp, pen = (float(x) for x in params[r])
            gen = []
            if penalty_ids is not None:
                gen = penalty_ids[int(penalty_offsets[r]):int(penalty_offsets[r + 1])].tolist()
            u = philox_uniform(int(seeds[r, 0]), int(seeds[r, 1]))
            tok, lp, _, _ = sample_row(logits[r].cpu(), t, int(k), p, mp, pen, gen, u)
            out_tokens[r] = tok
            out_logprobs[r] = lp
