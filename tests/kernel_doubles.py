"""A stand-in for the HIP kernel library, written with torch tensor operations.

It exists so that everything above the kernels (cache manager, step function,
scheduler, engine, replay) can be exercised on a machine without a GPU, the way
the reference's tests swap its Python oracle in for its CUDA kernel
(tests/test_engine.py:82-101 of the reference).  It is test code: the product
never imports it and has no path that computes without the HIP library.

Each method has the signature and the contract of the method of the same name of
`mini_llm_runtime_amd.kernels.ops.HipOps`.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from mini_llm_runtime_amd.kernels.pending import NormedDelta


class TorchOps:
    def __init__(self, dtype: torch.dtype = torch.float32, device: str = "cpu") -> None:
        self.dtype = dtype
        self.device = torch.device(device)
        self.calls: dict[str, int] = {}

    def _count(self, name: str) -> None:
        self.calls[name] = self.calls.get(name, 0) + 1

    # residual stream ------------------------------------------------------------------
    def embedding(self, table: torch.Tensor, ids: torch.Tensor, out_dtype=None) -> torch.Tensor:
        self._count("embedding")
        return table[ids.long()].to(out_dtype or torch.float32)

    def settle(self, h):
        if isinstance(h, NormedDelta):
            y = self._sum(h.y)
            return h.weight.float() * (y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + h.eps))
        return h

    @staticmethod
    def _sum(y):
        return y.float().sum(0) if y.dim() == 3 else y.float()

    def add_normed(self, x, y, weight, eps, next_weight=None, next_eps=0.0, cast=False):
        self._count("add_normed")
        assert x.dtype == torch.float32
        x += self.settle(NormedDelta(y, weight, eps))
        if next_weight is not None:
            return (next_weight.float() * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + next_eps))).to(self.dtype)
        return x.to(self.dtype) if cast else None

    def rmsnorm(self, x, weight, eps, delta=None):
        self._count("rmsnorm")
        assert x.dtype == torch.float32
        if isinstance(delta, NormedDelta):
            return self.add_normed(x, delta.y, delta.weight, delta.eps, next_weight=weight, next_eps=eps)
        if delta is not None:
            x += delta.float().sum(0) if delta.dim() == 3 else delta.float()
        variance = x.pow(2).mean(-1, keepdim=True)
        return (weight.float() * (x * torch.rsqrt(variance + eps))).to(self.dtype)

    def add_(self, x, delta):
        delta = self.settle(delta)
        x += self._sum(delta) if delta.dim() == x.dim() + 1 else delta.float()

    def scale_softcap_(self, x, scale=1.0, cap=None):
        x *= scale
        if cap is not None:
            x.copy_(cap * torch.tanh(x / cap))

    def gather_rows(self, x, rows):
        if isinstance(x, NormedDelta):
            return NormedDelta(self.gather_rows(x.y, rows), x.weight, x.eps)
        return (x[:, rows.long()] if x.dim() == 3 else x[rows.long()]).contiguous()

    # matrix products ---------------------------------------------------------------------
    def linear(
        self, x, weight, bias=None, out_dtype=None, kernel="auto", swiglu=False, partial_sums=False, for_stream=False,
        activation=None, multiply=None, clamped_glu=None, multiply_rows=None,
    ):
        self._count("linear")
        y = x.float() @ weight.float().t()
        if bias is not None:
            y = y + bias.float()
        if activation == "relu2":
            y = torch.clamp(y, min=0.0) ** 2
        elif activation == "sigmoid":
            y = torch.sigmoid(y)
        elif activation == "gelu_tanh":
            y = 0.5 * y * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (y + 0.044715 * y**3)))
        elif activation is not None:
            raise ValueError(activation)
        if multiply is not None:
            y = y * (multiply.float() if multiply_rows is None else multiply[multiply_rows.long()].float())
        if clamped_glu is not None:  # rows woven like swiglu's, the bias with them
            limit, alpha = clamped_glu
            quads = y.view(y.shape[0], -1, 4)
            gate = quads[..., :2].clamp(max=limit)
            up = quads[..., 2:].clamp(-limit, limit)
            y = (gate * torch.sigmoid(alpha * gate) * (up + 1.0)).reshape(y.shape[0], -1)
        if swiglu:  # rows of weight: gate 2j, gate 2j+1, up 2j, up 2j+1
            quads = y.view(y.shape[0], -1, 4)
            gate, up = quads[..., :2], quads[..., 2:]
            y = (gate * torch.sigmoid(gate) * up).reshape(y.shape[0], -1)
        return y.to(out_dtype or self.dtype)

    def silu_mul(self, gate_up):
        inter = gate_up.shape[1] // 2
        g = gate_up[:, :inter].float()
        u = gate_up[:, inter:].float()
        return (g * torch.sigmoid(g) * u).to(self.dtype)

    # positions and cache --------------------------------------------------------------------
    def rope_table(self, positions, inv_freq, amplitude=1.0):
        ang = positions.double()[:, None] * inv_freq.double()[None, :]
        return (ang.cos() * amplitude).float(), (ang.sin() * amplitude).float()

    def glu_clamped(self, sums, limit, alpha=1.702):
        self._count("glu_clamped")
        inter = sums.shape[1] // 2
        g = sums[:, :inter].float().clamp(max=limit)
        u = sums[:, inter:].float().clamp(-limit, limit)
        return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(self.dtype)

    @staticmethod
    def _rotate(x, rotation):  # x [T, n, d] float32; the first r dims in two halves
        if rotation is None:
            return x
        cos, sin, r = rotation
        half = r // 2
        a, b = x[..., :half], x[..., half:r]
        c, s = cos[:, None, :], sin[:, None, :]
        return torch.cat([a * c - b * s, b * c + a * s, x[..., r:]], dim=-1)

    def latent_prepare(
        self, projected, *, heads, head_dim, rot_dim, kv_rank, own_cache, gated, norm_weight, eps, rotation, slot_mapping,
        key_pages, value_pages, block_size, kernel_dim, queries=None,
    ):
        self._count("latent_prepare")
        tokens = projected.shape[0]
        p = projected.float()
        if queries is not None:  # the query sums come from a product of their own
            q = queries.float().view(tokens, heads, head_dim + rot_dim)
            at = 0
        else:
            q = p[:, : heads * (head_dim + rot_dim)].view(tokens, heads, head_dim + rot_dim)
            at = heads * (head_dim + rot_dim)
        q_plain = q[..., :head_dim].reshape(tokens, heads * head_dim).to(self.dtype)
        q_latent = torch.zeros(tokens, heads, kernel_dim, dtype=torch.float32)
        q_latent[..., kv_rank : kv_rank + rot_dim] = self._rotate(q[..., head_dim:], rotation)
        if own_cache:
            c = p[:, at : at + kv_rank]
            c = norm_weight.float() * (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps))
            r = self._rotate(p[:, None, at + kv_rank : at + kv_rank + rot_dim], rotation)[:, 0]
            at += kv_rank + rot_dim
            row = torch.zeros(tokens, kernel_dim, dtype=torch.float32)
            row[:, :kv_rank] = c
            row[:, kv_rank : kv_rank + rot_dim] = r
            value = torch.zeros(tokens, kernel_dim, dtype=torch.float32)
            value[:, :kv_rank] = c
            slots = slot_mapping.long()
            ok = slots >= 0
            page, off = slots[ok] // block_size, slots[ok] % block_size
            key_pages[page, 0, off, :] = row[ok].to(key_pages.dtype)
            value_pages[page, 0, :, off] = value[ok].to(value_pages.dtype)
        gate = torch.sigmoid(p[:, at : at + heads]) if gated else None
        return q_plain, q_latent.view(tokens, heads * kernel_dim).to(self.dtype), gate

    def heads_linear(self, x, weight, *, in_stride, out=None, out_stride=None, row_scale=None):
        self._count("heads_linear")
        heads, n, k = weight.shape
        tokens = x.shape[0]
        xin = x.view(tokens, heads, in_stride)[..., :k].float()
        y = torch.einsum("thk,hnk->thn", xin, weight.float())
        if row_scale is not None:
            y = y * row_scale.float()[..., None]
        if out is None:
            return y.reshape(tokens, heads * n).to(self.dtype)
        out.view(tokens, heads, out_stride)[..., :n] = y.to(out.dtype)
        return out

    def retention_scan(
        self, projected, state, read_rows, write_rows, ctx, *, heads, head_dim, value_dim, decay, key_scale, rotation,
        chunked=None,
    ):
        self._count("retention_scan")
        tokens = projected.shape[0]
        p = projected.float()
        qk = heads * head_dim
        q = self._rotate(p[:, :qk].view(tokens, heads, head_dim), rotation)
        k = self._rotate(p[:, qk : 2 * qk].view(tokens, heads, head_dim), rotation) * key_scale
        v = p[:, 2 * qk : 2 * qk + heads * value_dim].view(tokens, heads, value_dim)
        out = torch.zeros(tokens, heads, value_dim, dtype=torch.float32)
        for r in range(ctx.num_entries):
            a, b = int(ctx.cu_q[r]), int(ctx.cu_q[r + 1])
            s = state[int(read_rows[r])].float().clone() if int(ctx.q_starts[r]) > 0 else torch.zeros_like(state[0])
            for t in range(a, b):
                s = decay.float()[:, None, None] * s + k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", s, q[t])
            state[int(write_rows[r])] = s
        return out.view(tokens, heads * value_dim)

    def retention_gate(
        self, retained, projected, *, heads, value_dim, gate_offset, eps, norm_weight=None, scale=1.0, out=None, column=0,
        gate="silu",
    ):
        self._count("retention_gate")
        tokens = retained.shape[0]
        o = retained.float().view(tokens, heads, value_dim)
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        if norm_weight is not None:  # one weight for all heads, or one over all heads side by side
            o = o * (norm_weight.float().view(heads, value_dim) if norm_weight.numel() == heads * value_dim else norm_weight.float())
        z = projected[:, gate_offset : gate_offset + heads * value_dim].float()
        act = torch.sigmoid(z) if gate == "sigmoid" else z * torch.sigmoid(z)
        y = (o.reshape(tokens, heads * value_dim) * act * scale).to(self.dtype)
        if out is None:
            return y
        out[:, column : column + heads * value_dim] = y
        return out

    # parts that run side by side ---------------------------------------------------------------
    def short_conv(self, h, weight, state, read_rows, write_rows, ctx, *, add_input=True):
        self._count("short_conv")
        taps = weight.shape[1]
        carried = taps - 1
        w = weight.float()
        out = torch.zeros_like(h, dtype=torch.float32)
        for r in range(ctx.num_entries):
            a, b = int(ctx.cu_q[r]), int(ctx.cu_q[r + 1])
            before = torch.zeros(carried, h.shape[1])
            if carried and int(ctx.q_starts[r]) > 0:
                before = state[int(read_rows[r])].float().clone()
            seq = torch.cat([before, h[a:b].float()])
            for j in range(taps):
                out[a:b] += w[:, j] * seq[j : j + (b - a)]
            if add_input:
                out[a:b] += h[a:b].float()
            if carried:
                state[int(write_rows[r])] = seq[seq.shape[0] - carried :]
        return out.to(self.dtype)

    def qk_norm_rope_write(
        self, projected, q_norm, k_norm, eps, head_scale, rotation, slot_mapping, key_pages, value_pages, *, num_heads,
        num_kv_heads, dim, value_dim, head_dim, block_size, gated=False, projected_column=0,
    ):
        self._count("qk_norm_rope_write")
        tokens = projected.shape[0]
        p = projected.float()[:, projected_column:]
        qs, ks, vs = num_heads * dim, num_kv_heads * dim, num_kv_heads * value_dim
        q, k, v = p[:, :qs], p[:, qs : qs + ks], p[:, qs + ks : qs + ks + vs]
        if q_norm is not None:
            q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()
        if k_norm is not None:
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm.float()
        q = self._rotate(q.reshape(tokens, num_heads, dim), rotation)
        k = self._rotate(k.reshape(tokens, num_kv_heads, dim), rotation)
        if head_scale is not None:
            q = q * head_scale.float()[None, :, None]
        q_out = torch.zeros(tokens, num_heads, head_dim)
        q_out[..., :dim] = q
        k_out = torch.zeros(tokens, num_kv_heads, head_dim)
        k_out[..., :dim] = k
        v_out = torch.zeros(tokens, num_kv_heads, head_dim)
        v_out[..., :value_dim] = v.reshape(tokens, num_kv_heads, value_dim)
        slots = slot_mapping.long()
        ok = slots >= 0
        page, off = slots[ok] // block_size, slots[ok] % block_size
        key_pages[page, :, off, :] = k_out[ok].to(key_pages.dtype)
        value_pages[page, :, :, off] = v_out[ok].to(value_pages.dtype)
        gate = torch.sigmoid(p[:, qs + ks + vs : qs + ks + vs + num_heads]) if gated else None
        return q_out.reshape(tokens, num_heads * head_dim).to(self.dtype), gate

    def pool_kv_write(
        self, key_pages, value_pages, block_table, pooled_slots, pooled_keys, pooled_values, ctx, *, num_kv_heads, head_dim,
        block_size, pool,
    ):
        self._count("pool_kv_write")
        table = block_table.long()
        for t in range(pooled_slots.shape[0]):
            slot = int(pooled_slots[t])
            if slot < 0:
                continue
            p = int(ctx.positions[t])
            idx = torch.arange(p - pool + 1, p + 1)
            page = table[int(ctx.token_entry[t]), idx // block_size]
            assert (page >= 0).all(), "a run is pooled from pages that are not there"
            k = key_pages[page, :, idx % block_size, :].float().mean(0)  # [Hkv, d]
            v = value_pages[page, :, :, idx % block_size].float().mean(0)
            pooled_keys[slot // block_size, :, slot % block_size, :] = k.to(pooled_keys.dtype)
            pooled_values[slot // block_size, :, :, slot % block_size] = v.to(pooled_values.dtype)

    def scale_heads(self, attended, gate, *, heads, head_dim, out_dim, scale=1.0, out=None, column=0):
        self._count("scale_heads")
        tokens = attended.shape[0]
        y = attended.float().view(tokens, heads, head_dim)[..., :out_dim] * scale
        if gate is not None:
            y = y * gate.float()[:, :, None]
        y = y.reshape(tokens, heads * out_dim).to(self.dtype)
        if out is None:
            return y
        out[:, column : column + heads * out_dim] = y
        return out

    def gla_scan(
        self, projected, state, read_rows, write_rows, ctx, *, heads, head_dim, value_dim, decay_weight, decay_bias,
        low_offset, tau, q_scale, by_runs=None, projected_column=0,
    ):
        self._count("gla_scan")
        tokens = projected.shape[0]
        p = projected.float()[:, projected_column:]
        qk = heads * head_dim
        q = p[:, :qk].view(tokens, heads, head_dim) * q_scale
        k = p[:, qk : 2 * qk].view(tokens, heads, head_dim)
        v = p[:, 2 * qk : 2 * qk + heads * value_dim].view(tokens, heads, value_dim)
        rank = decay_weight.shape[1]
        z = p[:, low_offset : low_offset + rank] @ decay_weight.float().T
        if decay_bias is not None:
            z = z + decay_bias.float()
        alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(tokens, heads, head_dim)
        out = torch.zeros(tokens, heads, value_dim, dtype=torch.float32)
        for r in range(ctx.num_entries):
            a, b = int(ctx.cu_q[r]), int(ctx.cu_q[r + 1])
            s = state[int(read_rows[r])].float().clone() if int(ctx.q_starts[r]) > 0 else torch.zeros_like(state[0])
            for t in range(a, b):
                s = alpha[t][:, :, None] * s + k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", s, q[t])
            state[int(write_rows[r])] = s
        return out.view(tokens, heads * value_dim)

    def rope_kv_write(
        self, qkv, rotation, slot_mapping, key_pages, value_pages, *, num_heads, num_kv_heads, head_dim, block_size, write=True
    ):
        self._count("rope_kv_write")
        tokens = qkv.shape[0]
        qs = num_heads * head_dim
        ks = num_kv_heads * head_dim
        q = qkv[:, :qs].view(tokens, num_heads, head_dim)
        k = qkv[:, qs : qs + ks].view(tokens, num_kv_heads, head_dim)
        v = qkv[:, qs + ks :].view(tokens, num_kv_heads, head_dim)
        if rotation is not None:
            cos, sin, r = rotation
            half = r // 2
            for t in (q, k):
                a = t[..., :half].float().clone()
                b = t[..., half:r].float().clone()
                c = cos[:, None, :]
                s = sin[:, None, :]
                t[..., :half] = (a * c - b * s).to(t.dtype)
                t[..., half:r] = (b * c + a * s).to(t.dtype)
        if write:
            slots = slot_mapping.long()
            ok = slots >= 0
            page = slots[ok] // block_size
            off = slots[ok] % block_size
            key_pages[page, :, off, :] = k[ok]
            value_pages[page, :, :, off] = v[ok]

    def qkv_rope_write(self, x, weight, bias, rotation, slot_mapping, key_pages, value_pages, **sizes):
        qkv = self.linear(x, weight, bias)
        self.rope_kv_write(qkv, rotation, slot_mapping, key_pages, value_pages, **sizes)
        return qkv

    def paged_attention(
        self, qkv, key_pages, value_pages, block_table, ctx, *, num_heads, num_kv_heads, head_dim, block_size, scale, window,
        defer_merge=False, plan=None, chunk=None, sinks=None, pooled=None, score_bias=None,
    ):
        self._count("paged_attention")
        tokens = qkv.shape[0]
        group = num_heads // num_kv_heads
        q = qkv[:, : num_heads * head_dim].view(tokens, num_heads, head_dim).float()
        out = torch.zeros(tokens, num_heads, head_dim, dtype=torch.float32, device=qkv.device)
        table = block_table.long()
        for t in range(tokens):
            r = int(ctx.token_entry[t])
            p = int(ctx.positions[t])
            first = 0 if window is None else max(0, p - window + 1)
            if chunk is not None:
                first = p // chunk * chunk
            idx = torch.arange(first, p + 1)
            page = table[r, idx // block_size]
            assert (page >= 0).all(), "attention would read a page that is not there"
            k = key_pages[page, :, idx % block_size, :].float()  # [n, Hkv, d]
            v = value_pages[page, :, :, idx % block_size].float()
            if pooled is not None and p - window >= 0:  # the runs that end at or before p - window, through their means
                pk, pv, ptable, pool = pooled
                runs = torch.arange((p - window + 1) // pool)
                ppage = ptable.long()[r, runs // block_size]
                assert (ppage >= 0).all(), "attention would read a pooled page that is not there"
                k = torch.cat([pk[ppage, :, runs % block_size, :].float(), k])
                v = torch.cat([pv[ppage, :, :, runs % block_size].float(), v])
            k = k.repeat_interleave(group, dim=1)
            v = v.repeat_interleave(group, dim=1)
            s = torch.einsum("hd,nhd->hn", q[t], k) * scale
            if score_bias is not None:  # no softmax: every key weighs by itself
                w = torch.sigmoid(s + score_bias.float()[:, None])
            elif sinks is not None:  # one more term of the denominator, with no key and no value
                top = torch.maximum(s.max(-1).values, sinks.float())
                e = torch.exp(s - top[:, None])
                w = e / (e.sum(-1) + torch.exp(sinks.float() - top))[:, None]
            else:
                w = torch.softmax(s, dim=-1)
            out[t] = torch.einsum("hn,nhd->hd", w, v)
        return out.reshape(tokens, num_heads * head_dim).to(self.dtype)

    # several residual streams ---------------------------------------------------------------------
    def streams_fill(self, x, streams):
        self._count("streams_fill")
        return x.float()[None].repeat(streams, 1, 1).contiguous()

    def streams_step(self, x, *, update=None, read_weights=None, norm_weight=None, eps=0.0, rows=None, want_sum=False):
        self._count("streams_step")
        assert x.dtype == torch.float32 and x.dim() == 3
        new = x
        if update is not None:
            y, mix, write = update
            y = self._sum(self.settle(y))
            new = torch.einsum("st,snw->tnw", mix.float(), x) + write.float()[:, None, None] * y[None]
            if rows is None:
                x.copy_(new)
        if rows is not None:
            new = new[:, rows.long()]
        u = new.sum(0) if read_weights is None else torch.einsum("s,snw->nw", read_weights.float(), new)
        h = None
        if norm_weight is not None:
            h = (norm_weight.float() * (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps))).to(self.dtype)
        return h, (u if want_sum else None)

    def head_norm_rope_write(
        self, projected, *, heads, kv_heads, head_dim, value_dim, kernel_dim, eps, rotation, slot_mapping, key_pages,
        value_pages, block_size, gated=False, keep_values=False, first_values=None, mix_weight=None,
    ):
        self._count("head_norm_rope_write")
        tokens = projected.shape[0]
        p = projected.float()
        a, b = heads * head_dim, (heads + kv_heads) * head_dim
        c = b + kv_heads * value_dim

        def unit(x):
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)

        q = unit(self._rotate(p[:, :a].view(tokens, heads, head_dim), rotation))
        k = unit(self._rotate(p[:, a:b].view(tokens, kv_heads, head_dim), rotation))
        v = unit(p[:, b:c].view(tokens, kv_heads, value_dim))
        kept = v.reshape(tokens, kv_heads * value_dim).clone() if keep_values else None
        if first_values is not None:
            w = mix_weight.float()[0]
            v = (1.0 - w) * v + w * first_values.float().view(tokens, kv_heads, value_dim)
        q_out = torch.zeros(tokens, heads, kernel_dim)
        q_out[..., :head_dim] = q
        k_row = torch.zeros(tokens, kv_heads, kernel_dim)
        k_row[..., :head_dim] = k
        v_row = torch.zeros(tokens, kv_heads, kernel_dim)
        v_row[..., :value_dim] = v
        slots = slot_mapping.long()
        ok = slots >= 0
        page, off = slots[ok] // block_size, slots[ok] % block_size
        key_pages[page, :, off, :] = k_row[ok].to(key_pages.dtype)
        value_pages[page, :, :, off] = v_row[ok].to(value_pages.dtype)
        gate = torch.sigmoid(p[:, c : c + heads]) if gated else None
        return q_out.view(tokens, heads * kernel_dim).to(self.dtype), gate, kept

    def matrix_memory_scan(
        self, projected, state, read_rows, write_rows, ctx, *, heads, head_dim, value_dim, offsets, cap, q_scale,
        in_runs=None,
    ):
        self._count("matrix_memory_scan")
        tokens = projected.shape[0]
        p = projected.float()
        qa, ka, va, ia, fa = offsets
        q = p[:, qa : qa + heads * head_dim].view(tokens, heads, head_dim) * q_scale
        k = p[:, ka : ka + heads * head_dim].view(tokens, heads, head_dim)
        v = p[:, va : va + heads * value_dim].view(tokens, heads, value_dim)
        gi = cap * torch.tanh(p[:, ia : ia + heads] / cap)
        gf = torch.nn.functional.logsigmoid(cap * torch.tanh(p[:, fa : fa + heads] / cap))
        out = torch.zeros(tokens, heads, value_dim, dtype=torch.float32)
        cells = head_dim * value_dim
        for r in range(ctx.num_entries):
            a, b = int(ctx.cu_q[r]), int(ctx.cu_q[r + 1])
            row = state[int(read_rows[r])].float().clone() if int(ctx.q_starts[r]) > 0 else torch.zeros_like(state[0])
            C = row[:, :cells].reshape(heads, head_dim, value_dim)
            n = row[:, cells : cells + head_dim].clone()
            m = row[:, cells + head_dim].clone()
            for t in range(a, b):
                m_new = torch.maximum(gf[t] + m, gi[t])
                keep, take = torch.exp(gf[t] + m - m_new), torch.exp(gi[t] - m_new)
                C = keep[:, None, None] * C + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
                n = keep[:, None] * n + take[:, None] * k[t]
                m = m_new
                below = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
                out[t] = torch.einsum("hdv,hd->hv", C, q[t]) / below[:, None]
            state[int(write_rows[r])] = torch.cat([C.reshape(heads, cells), n, m[:, None]], dim=1)
        return out.view(tokens, heads * value_dim)

    # routed experts ------------------------------------------------------------------------------
    def route_experts(self, logits, correction, *, top, groups, keep_groups, scale, scores="sigmoid", normalise=False):
        self._count("route_experts")
        tokens, experts = logits.shape
        s = torch.softmax(logits.float(), -1) if scores == "softmax" else torch.sigmoid(logits.float())
        c = s + correction.float()
        per = experts // groups
        ids = torch.empty(tokens, top, dtype=torch.int32)
        weights = torch.empty(tokens, top, dtype=torch.float32)
        for t in range(tokens):
            score = [sum(sorted(c[t, g * per : (g + 1) * per].tolist(), reverse=True)[:2]) for g in range(groups)]
            kept = sorted(range(groups), key=lambda g: (-score[g], g))[:keep_groups]
            allowed = [e for e in range(experts) if e // per in kept]
            chosen = sorted(allowed, key=lambda e: (-float(c[t, e]), e))[:top]
            total = sum(float(s[t, e]) for e in chosen) + 1e-20 if normalise else 1.0
            for j, e in enumerate(chosen):
                ids[t, j] = e
                weights[t, j] = s[t, e] / total * scale
        return ids.to(logits.device), weights.to(logits.device)

    def expert_products(self, h, up_weight, down_weight, ids, weights, *, experts, activation, pass_through=0):
        self._count("expert_products")
        tokens, hidden = h.shape
        top = ids.shape[1]
        up = up_weight.float().view(experts, -1, hidden)
        down = down_weight.float().view(experts, hidden, -1)
        out = torch.zeros(top, tokens, hidden, dtype=torch.float32, device=h.device)
        for t in range(tokens):
            for j in range(top):
                e = int(ids[t, j])
                if e >= experts:  # an expert without matrices: its input itself
                    assert e < experts + pass_through
                    out[j, t] = weights[t, j] * h[t].float()
                    continue
                z = up[e] @ h[t].float()
                if activation == "swiglu":
                    z = z.to(self.dtype).float()
                    half = z.shape[0] // 2
                    a = z[:half] * torch.sigmoid(z[:half]) * z[half:]
                else:
                    a = torch.clamp(z, min=0.0) ** 2 if activation == "relu2" else torch.sigmoid(z)
                out[j, t] = weights[t, j] * (down[e] @ a.to(self.dtype).float())
        return out

    # sampling ----------------------------------------------------------------------------------
    def sample(self, logits, temperature: Optional[torch.Tensor], uniform: Optional[torch.Tensor]):
        self._count("sample")
        greedy = torch.argmax(logits, dim=-1).to(torch.int32)
        if temperature is None:
            return greedy
        out = greedy.clone()
        for i in range(logits.shape[0]):
            t = float(temperature[i])
            if t > 0:
                z = logits[i].float()
                e = torch.exp((z - z.max()) / t)
                c = torch.cumsum(e, dim=0)
                target = float(uniform[i]) * float(c[-1])
                out[i] = min(int(torch.searchsorted(c, torch.tensor(target), right=True)), logits.shape[1] - 1)
        return out
