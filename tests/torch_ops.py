"""Plain torch twins of the HIP kernels, with the same call signatures and the same page layout.

Two uses: each is the reference its kernel is tested against on the GPU, and together they let
the tests drive the engine's step function, cache and scheduler on a CPU (the product has no CPU
path of its own; the tests pass this object in place of the kernel namespace).  Arithmetic is
float32 inside, like the kernels.
"""
from __future__ import annotations

import torch

from llmserver_amd.parts.attention import group_tiling  # noqa: F401  (kept for symmetry of imports)
from llmserver_amd.parts.kernel_namespace import KernelNamespace


class TorchOps(KernelNamespace):
    """``fused=True`` also offers the twins of the fused kernels (sum and norm folded into the few-row products, q/k
    norm, rotation and cache write inside the attention of single-token steps), for any type and size, so that the
    parts' fused dataflow runs on the CPU as it does on the GPU."""
    name = "torch"
    FUSED_ROWS = 16

    def __init__(self, fused: bool = False):
        self.fuse_stream_updates = fused
        self.fused = fused
        self.fused_calls = {"row_scale": 0, "into_stream": 0, "gated": 0, "decode_attention": 0, "partial_sums": 0}

    def preload(self, head_dims, dtype):
        pass

    # -- twins of the fused few-row products ------------------------------------------------------
    def row_scale_fits(self, x, weight, row_scale) -> bool:
        return self.fused and x.shape[1] == weight.shape[1] and 0 < x.shape[0] <= self.FUSED_ROWS

    @staticmethod
    def _scaled(y, row_scale, width):
        if row_scale is None:
            return y
        square_sums, eps = row_scale
        return y * torch.rsqrt(square_sums.float().sum(dim=1, keepdim=True) / width + eps)

    def linear_few_rows(self, x, weight, out=None, out_float32=False, rows_per_workgroup=0, row_scale=None):
        if not self.row_scale_fits(x, weight, row_scale):
            return None
        self.fused_calls["row_scale"] += row_scale is not None
        y = self._scaled(x.float() @ weight.float().t(), row_scale, x.shape[1])
        return y if (out_float32 or x.dtype == torch.float32) else y.to(x.dtype)

    def linear_into_stream(self, x, weight, resid, norm_weight, rows_per_workgroup=0, row_scale=None):
        if not self.row_scale_fits(x, weight, row_scale):
            return None
        self.fused_calls["into_stream"] += 1
        y = self._scaled(x.float() @ weight.float().t(), row_scale, x.shape[1]).to(x.dtype)
        stream = (resid.float() + y.float()).to(resid.dtype)
        weighted = (stream.float() * norm_weight).to(resid.dtype)
        squares = stream.float() ** 2
        parts = torch.stack([squares[:, i::3].sum(dim=1) for i in range(3)], dim=1)      # any split of the row will do
        return stream, weighted, parts

    def linear_gated(self, x, gate_up_weight, pairs_per_workgroup=0, row_scale=None, activation="silu"):
        beyond = self.fused and row_scale is None and 16 < x.shape[0] <= 32            # the kernel for more rows has no row scale
        if not beyond and not self.row_scale_fits(x, gate_up_weight, row_scale):
            return None
        self.fused_calls["gated"] += 1
        gate_up = self._scaled(x.float() @ gate_up_weight.float().t(), row_scale, x.shape[1])
        inter = gate_up.shape[1] // 2
        gate, up = gate_up[:, :inter], gate_up[:, inter:]
        return (self._activated(gate, activation) * up).to(x.dtype)

    def linear_partial_sums(self, x, weight, few_rows_too=False):
        if not self.fused or not (0 if few_rows_too else 16) < x.shape[0] <= 128:
            return None
        self.fused_calls["partial_sums"] += 1
        bounds = [0, x.shape[1] // 3, x.shape[1] // 2, x.shape[1]]                      # any split of the inner dimension
        return torch.stack([x[:, a:b].float() @ weight[:, a:b].float().t() for a, b in zip(bounds, bounds[1:])])

    def decode_fusion_fits(self, dtype, head_dim) -> bool:
        return self.fused

    def linear(self, x, weight, out=None, out_float32=False):
        y = (x.float() @ weight.float().t())
        y = y if (out_float32 or x.dtype == torch.float32) else y.to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def embedding(self, table, token_ids, out):
        out.copy_(table[token_ids.long()])

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None):
        if delta is not None and delta.dim() == 3:                                       # partial sums of the update
            delta = delta.sum(dim=0).to(resid.dtype)
        if rows is None:
            total = resid.float()
            if delta is not None:
                total = (total + delta.float()).to(resid.dtype)
                resid.copy_(total)
                total = total.float()
        else:
            index = rows.long()
            total = resid[index].float()
            if delta is not None:
                total = (total + delta[index].float()).to(resid.dtype).float()
        normed = total * torch.rsqrt(total.pow(2).mean(dim=-1, keepdim=True) + eps) * weight
        out.copy_(normed.to(out.dtype))

    @staticmethod
    def _activated(gate, activation):
        if activation == "silu":
            return gate * torch.sigmoid(gate)
        if activation == "gelu_tanh":
            return 0.5 * gate * (1.0 + torch.tanh(0.7978845608028654 * (gate + 0.044715 * gate ** 3)))
        raise ValueError(f"no twin for the activation {activation!r}")

    def swiglu(self, gate_up, out, activation="silu"):
        inter = out.shape[1]
        gate, up = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        out.copy_((self._activated(gate, activation) * up).to(out.dtype))

    def add_bias_(self, y, bias):
        y.copy_((y.float() + bias).to(y.dtype))

    def rotary_table(self, positions, inv_freq):
        angles = positions.float()[:, None] * inv_freq[None, :]
        return torch.cat([torch.cos(angles), torch.sin(angles)], dim=1)

    def qk_norm_rope_kv_write(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin,
                              page_size, n_q, n_kv, head_dim, write_cache=True):
        n = qkv.shape[0]
        heads = qkv.view(n, n_q + 2 * n_kv, head_dim)
        qk = heads[:, :n_q + n_kv].float()
        if q_weight is not None:
            weight = torch.cat([q_weight.expand(n_q, -1), k_weight.expand(n_kv, -1)], dim=0)
            qk = qk * torch.rsqrt(qk.pow(2).mean(dim=-1, keepdim=True) + eps) * weight
        if cos_sin is not None:
            half = head_dim // 2
            cos, sin = cos_sin[:, None, :half], cos_sin[:, None, half:]
            x1, x2 = qk[..., :half], qk[..., half:]
            qk = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
        heads[:, :n_q] = qk[:, :n_q].to(qkv.dtype)
        if not write_cache:
            return
        pos = positions.long()
        pages = table.long()[token_row.long(), pos // page_size]
        slots = pos % page_size
        keys[pages, :, slots, :] = qk[:, n_q:].to(keys.dtype)
        values[pages, :, :, slots] = heads[:, n_q + n_kv:].to(values.dtype)

    def paged_attention(self, qkv, out, keys, values, table, row_start, row_len, row_ctx, plan, scale, window, page_size,
                        n_q, n_kv, head_dim, ctx, decode_fusion=None, sinks=None, softcap=None):
        """Per request row: gather its keys/values through the block table, one softmax over all
        keys a query may see (no tiles, no splits).  ``decode_fusion``: the step's rows bring one token each and
        ``qkv`` is the raw projection, which is left as it is."""
        if decode_fusion is not None:
            self.fused_calls["decode_attention"] += 1
            q_weight, k_weight, eps, cos_sin, write_cache = decode_fusion
            rows = table.shape[0]
            assert qkv.shape[0] == rows and all(int(n) == 1 for n in row_len)
            qkv = qkv.clone()
            token_row = torch.arange(rows, dtype=torch.int32, device=qkv.device)
            positions = (row_ctx - 1).to(torch.int32)
            self.qk_norm_rope_kv_write(qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin, page_size,
                                       n_q, n_kv, head_dim, write_cache)
        n = qkv.shape[0]
        q_all = qkv.view(n, -1, head_dim)[:, :n_q].float()
        group = n_q // n_kv
        for row in range(table.shape[0]):
            start, length, ctx_len = int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            first = 0 if not window else max(0, ctx_len - length - window + 1)
            place = torch.arange(first, ctx_len, device=qkv.device)
            pages = table[row].long()[place // page_size]
            k = keys[pages, :, place % page_size, :].float()            # [keys, n_kv, d]
            v = values[pages, :, :, place % page_size].float()          # [keys, n_kv, d]
            q = q_all[start:start + length]                               # [len, n_q, d]
            k = k.repeat_interleave(group, dim=1)
            v = v.repeat_interleave(group, dim=1)
            scores = torch.einsum("qhd,khd->hqk", q, k) * scale
            if softcap:
                scores = softcap * torch.tanh(scores / softcap)
            q_pos = torch.arange(ctx_len - length, ctx_len, device=qkv.device)
            hidden = place[None, :] > q_pos[:, None]
            if window:
                hidden = hidden | (place[None, :] <= q_pos[:, None] - window)
            scores = scores.masked_fill(hidden[None], float("-inf"))
            if sinks is None:
                weights = torch.softmax(scores, dim=-1)
            else:
                top = torch.maximum(scores.max(dim=-1).values, sinks.float()[:, None])
                weights = torch.exp(scores - top[..., None])
                weights = weights / (weights.sum(dim=-1) + torch.exp(sinks.float()[:, None] - top))[..., None]
            result = torch.einsum("hqk,khd->qhd", weights, v)
            out[start:start + length] = result.reshape(length, n_q * head_dim).to(out.dtype)

    # -- a 32-bit residual stream -----------------------------------------------------------------------
    @staticmethod
    def _rms(x, eps):
        return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)

    def embedding_norm(self, table, token_ids, weight, eps, out):
        out.copy_(self._rms(table[token_ids.long()].float(), eps) * weight)

    def embedding_wide(self, table, token_ids, out, scale=1.0):
        out.copy_(table[token_ids.long()].float() * scale)        # (several streams: the rows once for each)

    def streams_read(self, streams, read, weight, eps, out, rows=None):
        picked = streams if rows is None else streams[:, rows.long()]
        out.copy_((self._rms((picked * read[:, None, None]).sum(dim=0), eps) * weight).to(out.dtype))

    def streams_update(self, streams, y, mix, write, next_read=None, next_weight=None, next_eps=0.0, normed=None):
        new = torch.einsum("st,snw->tnw", mix, streams) + write[:, None, None] * y.float()[None]
        streams.copy_(new)
        if next_read is not None:
            self.streams_read(streams, next_read, next_weight, next_eps, normed)

    def linear_activated(self, x, weight, activation):
        z = x.float() @ weight.float().t()
        return (torch.relu(z) ** 2 if activation == "relu2" else self._activated(z, activation)).to(x.dtype)

    def activation_(self, x, activation):
        z = x.float()
        x.copy_((torch.relu(z) ** 2 if activation == "relu2" else self._activated(z, activation)).to(x.dtype))

    def norm_add_norm(self, x, y, weight, eps, out, next_weight=None, next_eps=0.0, normed=None, y2=None, scales=None):
        update = y.float() if y2 is None else scales[0] * y.float() + scales[1] * y2.float()
        total = x + self._rms(update, eps) * weight
        out.copy_(total)
        if next_weight is not None:
            normed.copy_((self._rms(total, next_eps) * next_weight).to(normed.dtype))

    def norm_rows(self, x, rows, weight, eps, out):
        picked = x if rows is None else x[rows.long()]
        out.copy_((self._rms(picked.float(), eps) * weight).to(out.dtype))

    def short_conv(self, x, weight, state, state_slots, token_row, positions, row_start, out, keep=False):
        taps = weight.shape[1]
        result = x.clone()
        for t in range(x.shape[0]):
            row, position = int(token_row[t]), int(positions[t])
            first = position - (t - int(row_start[row]))            # position of the row's first token in this step
            for j in range(taps):
                back = taps - 1 - j
                place = position - back
                if place < 0:
                    continue
                if place >= first:
                    value = x[t - back]
                else:
                    value = state[int(state_slots[row]), taps - 1 - (first - place)]
                result[t] += weight[:, j] * value
        out.copy_(result.to(out.dtype))
        if keep:
            assert x.shape[0] == len(row_start)
            for t in range(x.shape[0]):
                slot = int(state_slots[int(token_row[t])])
                state[slot] = torch.cat([state[slot, 1:], x[t:t + 1]], dim=0)

    def short_conv_keep(self, x, state, state_slots, row_start, row_len, row_ctx):
        kept = state.shape[1]
        for row in range(len(row_len)):
            slot, start, count, end = int(state_slots[row]), int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            first = end - count
            old = state[slot].clone()
            for k in range(kept):
                place = end - kept + k
                if place >= first:
                    state[slot, k] = x[start + place - first]
                elif place >= 0:
                    state[slot, k] = old[k + count]
                else:
                    state[slot, k] = 0

    def scaled_norm_add(self, x, y, weight, scale, eps, out, rounded=None, history=None, before=0, mix=None):
        s = x + self._rms(y.float(), eps) * weight * (1.0 if scale is None else scale)
        if history is not None:
            history[before] = s
            s = (history[:before + 1] * mix[:before + 1, None, None]).sum(dim=0)
        out.copy_(s)
        if rounded is not None:
            rounded.copy_(s.to(rounded.dtype))

    # -- general preparation of queries, keys and values -------------------------------------------------
    def qkv_prepare(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin, page_size,
                    n_q, n_kv, dim, value_dim, out_q, write_cache=True, pairing="neighbours", value_share=1):
        n, width = qkv.shape[0], keys.shape[-1]
        q = qkv[:, :n_q * dim].float().view(n, n_q, dim)
        if not write_cache and qkv.shape[1] == n_q * dim:            # a layer that reads another's pages brings queries only
            out_q.copy_(torch.nn.functional.pad(q, (0, width - dim)).reshape(n, n_q * width).to(out_q.dtype))
            assert q_weight is None and cos_sin is None
            return
        k = qkv[:, n_q * dim:(n_q + n_kv) * dim].float().view(n, n_kv, dim)
        v = qkv[:, (n_q + n_kv) * dim:].float().view(n, n_kv // value_share, value_dim).repeat_interleave(value_share, dim=1)
        if q_weight is not None:
            q, k = self._rms(q, eps) * q_weight, self._rms(k, eps) * k_weight
        if cos_sin is not None:
            pairs = cos_sin.shape[1] // 2
            cos, sin = cos_sin[:, None, :pairs], cos_sin[:, None, pairs:]

            def turned(x):
                if pairing == "halves":
                    a, b = x[..., :pairs], x[..., pairs:2 * pairs]
                    return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., 2 * pairs:]], dim=-1)
                a, b = x[..., 0:2 * pairs:2], x[..., 1:2 * pairs:2]
                return torch.cat([torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1).flatten(-2), x[..., 2 * pairs:]], dim=-1)
            q, k = turned(q), turned(k)
        full = torch.zeros((n, n_q, width), dtype=torch.float32, device=qkv.device)
        full[..., :dim] = q
        out_q.copy_(full.view(n, n_q * width).to(out_q.dtype))
        if not write_cache:
            return
        pos = positions.long()
        pages = table.long()[token_row.long(), pos // page_size]
        slots = pos % page_size
        key_rows = torch.zeros((n, n_kv, width), dtype=torch.float32, device=qkv.device)
        key_rows[..., :dim] = k
        value_rows = torch.zeros((n, n_kv, width), dtype=torch.float32, device=qkv.device)
        value_rows[..., :value_dim] = v
        keys[pages, :, slots, :] = key_rows.to(keys.dtype)
        values[pages, :, :, slots] = value_rows.to(values.dtype)

    # -- recurrent mixers --------------------------------------------------------------------------------
    def token_shift(self, h, mu, state, offset, state_slots, token_row, positions, row_start, out, keep=False):
        width = h.shape[1]
        before = torch.zeros_like(h, dtype=torch.float32)
        for t in range(h.shape[0]):
            row = int(token_row[t])
            if int(positions[t]) == 0:
                continue
            before[t] = h[t - 1].float() if t > int(row_start[row]) else state[int(state_slots[row]), offset:offset + width]
        wide = h.float()
        out.copy_((wide[None] + (before - wide)[None] * mu[:, None, :]).to(out.dtype))
        if keep:
            assert h.shape[0] == len(row_start)
            for t in range(h.shape[0]):
                state[int(state_slots[int(token_row[t])]), offset:offset + width] = h[t].float()

    def token_shift_keep(self, h, state, offset, state_slots, row_start, row_len):
        width = h.shape[1]
        for row in range(len(row_len)):
            if int(row_len[row]) > 0:
                state[int(state_slots[row]), offset:offset + width] = h[int(row_start[row]) + int(row_len[row]) - 1].float()

    def batched_linear(self, x, weights):
        return torch.bmm(x.float(), weights.float().transpose(1, 2)).to(x.dtype)

    def tanh_(self, x):
        x.copy_(torch.tanh(x.float()).to(x.dtype))

    def linear_recurrence(self, q, k, v, decay, decay_bias, decay_mode, tau, bonus, q_scale, state, offset, state_slots,
                          row_start, row_len, row_ctx, out, heads, dim, value_dim):
        z = decay.float() + (decay_bias if decay_bias is not None else 0.0)
        if decay_mode == "sigmoid_root":
            factor = torch.exp(torch.nn.functional.logsigmoid(z) / tau)
        elif decay_mode == "double_exp":
            factor = torch.exp(-torch.exp(z))
        else:
            raise ValueError(decay_mode)
        size = heads * dim * value_dim
        for row in range(len(row_len)):
            start, count, end = int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            if count <= 0:
                continue
            slot = int(state_slots[row])
            matrix = state[slot, offset:offset + size].view(heads, dim, value_dim).clone()
            if end - count == 0:
                matrix.zero_()
            for t in range(start, start + count):
                qt = q[t].float().view(heads, dim) * q_scale
                kv = k[t].float().view(heads, dim)[:, :, None] * v[t].float().view(heads, value_dim)[:, None, :]
                d = factor[t].view(heads, dim)[:, :, None]
                if bonus is None:
                    matrix = d * matrix + kv
                    out[t] = torch.einsum("hdv,hd->hv", matrix, qt).reshape(-1)
                else:
                    out[t] = torch.einsum("hdv,hd->hv", matrix + bonus[:, :, None] * kv, qt).reshape(-1)
                    matrix = d * matrix + kv
            state[slot, offset:offset + size] = matrix.reshape(-1)

    def heads_norm_gate(self, x, weight, weight_per_channel, eps, gate, out, heads, value_dim, gate_activation="silu", below=None, floor=0.0):
        n = x.shape[0]
        rows = x.float().view(n, heads, value_dim)
        if below is not None:
            rows = rows / (torch.maximum(below[..., 0].abs(), below[..., 1]) + floor)[..., None]
        normed = self._rms(rows, eps)
        normed = normed * (weight.view(heads, value_dim) if weight_per_channel else weight)
        g = gate.float().reshape(n, heads, value_dim)
        g = torch.sigmoid(g) if gate_activation == "sigmoid" else g * torch.sigmoid(g)
        out.copy_((normed * g).reshape(n, heads * value_dim).to(out.dtype))

    def matrix_memory_chunks(self, n_tokens, rows):
        return 0

    def matrix_memory(self, q, k, v, gates, cap, q_scale, state, state_slots, row_start, row_len, row_ctx, out, below, coefficients,
                      heads, dim, value_dim, run=None, sums=None):
        matrix_size, normaliser_size = heads * dim * value_dim, heads * dim
        log_in = cap * torch.tanh(gates[:, :heads].float() / cap)
        log_forget = torch.nn.functional.logsigmoid(cap * torch.tanh(gates[:, heads:].float() / cap))
        for row in range(len(row_len)):
            start, count, end = int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            if count <= 0:
                continue
            slot = int(state_slots[row])
            kept = state[slot].clone()
            if end - count == 0:
                kept.zero_()
            matrix = kept[:matrix_size].view(heads, dim, value_dim)
            normaliser = kept[matrix_size:matrix_size + normaliser_size].view(heads, dim)
            top = kept[matrix_size + normaliser_size:matrix_size + normaliser_size + heads]
            for t in range(start, start + count):
                qt, kt = q[t].float().view(heads, dim) * q_scale, k[t].float().view(heads, dim)
                new_top = torch.maximum(log_forget[t] + top, log_in[t])
                keep, take = torch.exp(log_forget[t] + top - new_top), torch.exp(log_in[t] - new_top)
                matrix = keep[:, None, None] * matrix + take[:, None, None] * kt[:, :, None] * v[t].float().view(heads, value_dim)[:, None, :]
                normaliser = keep[:, None] * normaliser + take[:, None] * kt
                top = new_top
                coefficients[t, :, 0], coefficients[t, :, 1] = keep, take
                below[t, :, 0], below[t, :, 1] = (normaliser * qt).sum(dim=-1), torch.exp(-top)
                out[t] = torch.einsum("hdv,hd->hv", matrix, qt).reshape(-1)
            state[slot, :matrix_size] = matrix.reshape(-1)
            state[slot, matrix_size:matrix_size + normaliser_size] = normaliser.reshape(-1)
            state[slot, matrix_size + normaliser_size:matrix_size + normaliser_size + heads] = top

    def scaled_sum(self, x, x_scale, y, y_scale, out):
        out.copy_((x_scale * x.float() + y_scale * y.float()).to(out.dtype))

    # -- attention over a shared latent ------------------------------------------------------------------
    inside = False          # True: the parts are told to let latent_prepare and gate_heads make the per-head products

    def latent_products_inside(self, n_tokens):
        return self.inside

    def latent_prepare(self, proj, q_latent, norm_weight, eps, cos_sin, keys, values, table, token_row, positions, page_size,
                       out_q, n_heads, dim, rot_dim, rank, write_cache=True, up_keys=None):
        n, width = proj.shape[0], keys.shape[-1]
        q = proj[:, :n_heads * (dim + rot_dim)].float().view(n, n_heads, dim + rot_dim)
        if q_latent is None:
            q_latent = torch.einsum("thd,hdr->htr", q[..., :dim], up_keys.float())
        down = proj[:, n_heads * (dim + rot_dim):n_heads * (dim + rot_dim) + rank + rot_dim].float()
        pairs = cos_sin.shape[1] // 2
        cos, sin = cos_sin[:, :pairs], cos_sin[:, pairs:]

        def turned(x):                                  # x [T, ..., rot_dim]
            shape = [n] + [1] * (x.dim() - 2) + [pairs]
            u, v = x[..., 0:2 * pairs:2], x[..., 1:2 * pairs:2]
            c, s = cos.view(shape), sin.view(shape)
            return torch.cat([torch.stack([u * c - v * s, v * c + u * s], dim=-1).flatten(-2), x[..., 2 * pairs:]], dim=-1)

        full = torch.zeros((n, n_heads, width), dtype=torch.float32, device=proj.device)
        full[..., :rank] = q_latent.float().transpose(0, 1)
        full[..., rank:rank + rot_dim] = turned(q[..., dim:])
        out_q.copy_(full.view(n, n_heads * width).to(out_q.dtype))
        if not write_cache:
            return
        row = torch.zeros((n, width), dtype=torch.float32, device=proj.device)
        row[:, :rank] = self._rms(down[:, :rank], eps) * norm_weight
        row[:, rank:rank + rot_dim] = turned(down[:, rank:])
        pos = positions.long()
        pages = table.long()[token_row.long(), pos // page_size]
        slots = pos % page_size
        keys[pages, 0, slots, :] = row.to(keys.dtype)
        values[pages, 0, :, slots] = row.to(values.dtype)

    def gate_heads(self, y, proj, gate_column, out, mixed=None, up_values=None, per_channel=False):
        if y is None:
            heads, rank, _ = up_values.shape
            rows = mixed.float().view(mixed.shape[0], heads, -1)[:, :, :rank]
            y = torch.einsum("thr,hrv->htv", rows, up_values.float())
        heads, n, v = y.shape
        if per_channel and gate_column >= 0:
            gate = torch.sigmoid(proj[:, gate_column:gate_column + heads * v].float()).view(n, heads, v)
            out.copy_((y.float().transpose(0, 1) * gate).reshape(n, heads * v).to(out.dtype))
            return
        gate = torch.sigmoid(proj[:, gate_column:gate_column + heads].float()) if gate_column >= 0 else torch.ones(n, heads, device=y.device)
        out.copy_((y.float().transpose(0, 1) * gate[..., None]).reshape(n, heads * v).to(out.dtype))

    # -- a block whose sublayers join the stream together; differential attention; the gated delta rule -----------------
    def gated_pair_update(self, x, gates, y1, scale1, y2, scale2, next_weight=None, next_eps=0.0, normed=None):
        width = x.shape[1]
        g = torch.sigmoid(gates.float())
        x += scale1 * g[:, :width] * y1.float()
        if y2 is not None:
            x += scale2 * g[:, width:] * y2.float()
        if next_weight is not None:
            normed.copy_((self._rms(x, next_eps) * next_weight).to(normed.dtype))

    def differential_heads(self, attended, lam, keep, eps, out, kv_heads, group, value_dim, row):
        n = attended.shape[0]
        maps = attended.float().view(n, kv_heads, 2, group, row)[..., :value_dim]
        d = maps[:, :, 0] - lam * maps[:, :, 1]
        out.copy_((self._rms(d, eps) * keep).reshape(n, kv_heads * group * value_dim).to(out.dtype))

    def delta_prepare(self, proj, taps, state, offset, state_slots, token_row, positions, row_start, out, kv_heads, heads, dim,
                      value_dim, q_scale, unit_eps, strength, decay, decay_scale, decay_bias, per_channel, out_strength, out_decay,
                      keep=False):
        out_strength.copy_(torch.sigmoid(strength.float()))
        step = torch.nn.functional.softplus(decay.float() + decay_bias)
        rate = torch.exp(decay_scale)
        out_decay.copy_(torch.exp(-(rate[None, :, None] * step.view(-1, heads, dim)).reshape(step.shape[0], -1) if per_channel else -rate * step))
        channels, count = taps.shape
        kept = count - 1
        x = proj[:, :channels].float()
        result = torch.zeros_like(x)
        for t in range(x.shape[0]):
            row, position = int(token_row[t]), int(positions[t])
            first = position - (t - int(row_start[row]))
            slot = int(state_slots[row])
            old = state[slot, offset:offset + kept * channels].view(kept, channels)
            for j in range(count):
                back = kept - j
                place = position - back
                if place < 0:
                    continue
                value = x[t - back] if place >= first else old[kept - (first - place)]
                result[t] += taps[:, j] * value
        result = result * torch.sigmoid(result)
        keys = kv_heads * dim
        for start in (0, keys):
            part = result[:, start:start + keys].view(-1, kv_heads, dim)
            part = part / torch.sqrt(part.pow(2).sum(dim=-1, keepdim=True) + unit_eps)
            result[:, start:start + keys] = (part * (q_scale if start == 0 else 1.0)).reshape(-1, keys)
        out.copy_(result)
        if keep and kept:
            assert x.shape[0] == len(row_start)
            for t in range(x.shape[0]):
                slot = int(state_slots[int(token_row[t])])
                old = state[slot, offset:offset + kept * channels].view(kept, channels)
                state[slot, offset:offset + kept * channels] = torch.cat([old[1:], x[t:t + 1]], dim=0).reshape(-1)

    def delta_conv_keep(self, proj, channels, taps, state, offset, state_slots, row_start, row_len, row_ctx):
        kept = taps - 1
        x = proj[:, :channels].float()
        for row in range(len(row_len)):
            slot, start, count, end = int(state_slots[row]), int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            if count <= 0:
                continue
            first = end - count
            old = state[slot, offset:offset + kept * channels].view(kept, channels).clone()
            new = torch.zeros_like(old)
            for k in range(kept):
                place = end - kept + k
                if place >= first:
                    new[k] = x[start + place - first]
                elif place >= 0:
                    new[k] = old[k + count]
            state[slot, offset:offset + kept * channels] = new.reshape(-1)

    def delta_rule(self, prepared, strength, decay, per_channel, state, offset, state_slots, row_start, row_len, row_ctx, out,
                   heads, kv_heads, dim, value_dim):
        blocks = -(-value_dim // 16)
        keys, size, repeat = kv_heads * dim, heads * dim * blocks * 16, heads // kv_heads
        beta = strength
        g = decay.view(-1, heads, dim)[..., None] if per_channel else decay[:, :, None, None]
        for row in range(len(row_len)):
            start, count, end = int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            if count <= 0:
                continue
            slot = int(state_slots[row])
            # (kept as blocks of 16 value columns, [heads, blocks, dim, 16])
            matrix = state[slot, offset:offset + size].view(heads, blocks, dim, 16).permute(0, 2, 1, 3).reshape(heads, dim, blocks * 16)[..., :value_dim].clone()
            if end - count == 0:
                matrix.zero_()
            for t in range(start, start + count):
                q = prepared[t, :keys].view(kv_heads, dim).repeat_interleave(repeat, dim=0)
                k = prepared[t, keys:2 * keys].view(kv_heads, dim).repeat_interleave(repeat, dim=0)
                v = prepared[t, 2 * keys:].view(heads, value_dim)
                matrix = matrix * g[t]
                u = beta[t][:, None] * (v - torch.einsum("hdv,hd->hv", matrix, k))
                matrix = matrix + k[:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", matrix, q).reshape(-1)
            kept = matrix.new_zeros((heads, dim, blocks * 16))           # (columns beyond the values are zeros)
            kept[..., :value_dim] = matrix
            state[slot, offset:offset + size] = kept.view(heads, dim, blocks, 16).permute(0, 2, 1, 3).reshape(-1)

    # -- routed experts ----------------------------------------------------------------------------------
    def route_experts(self, x, router, top, chosen, weights, scoring="softmax", groups=None, bias=None):
        logits = x.float() @ router.float().t()
        if bias is not None:
            logits = logits + bias
        if scoring == "softmax":
            best = torch.topk(logits, top, dim=-1)
            chosen.copy_(best.indices.to(chosen.dtype))
            weights.copy_(torch.softmax(best.values, dim=-1))
            return
        scores = torch.sigmoid(logits)
        allowed = scores
        if groups is not None:
            count, keep = groups
            per = scores.shape[1] // count
            grouped = scores.view(-1, count, per)
            group_scores = torch.topk(grouped, min(2, per), dim=-1).values.sum(dim=-1)
            kept = torch.zeros_like(group_scores, dtype=torch.bool)
            for _ in range(keep):                               # the best groups, the first of equal ones
                pick = group_scores.masked_fill(kept, float("-inf")).argmax(dim=-1, keepdim=True)
                kept.scatter_(1, pick, True)
            allowed = scores.masked_fill(~kept[:, :, None].expand(-1, -1, per).reshape(scores.shape), float("-inf"))
        for k in range(top):                                    # the largest scores, the first of equal ones
            pick = allowed.argmax(dim=-1, keepdim=True)
            chosen[:, k] = pick[:, 0].to(chosen.dtype)
            weights[:, k] = scores.gather(1, pick)[:, 0]
            allowed = allowed.scatter(1, pick, float("-inf"))

    def experts_gate_up(self, x, gate_up, chosen, hidden, activation="silu", limit=0.0):
        top, inter = chosen.shape[1], hidden.shape[1]
        for t in range(x.shape[0]):
            for s in range(top):
                both = gate_up[int(chosen[t, s])].float() @ x[t].float()
                gate, up = both[:inter], both[inter:]
                if activation == "clamped":
                    gate, up = gate.clamp(max=limit), up.clamp(min=-limit, max=limit)
                    hidden[t * top + s] = (gate * torch.sigmoid(1.702 * gate) * (up + 1.0)).to(hidden.dtype)
                else:
                    hidden[t * top + s] = (gate * torch.sigmoid(gate) * up).to(hidden.dtype)

    def experts_down(self, hidden, down, chosen, weights, out):
        top = chosen.shape[1]
        out.zero_()
        for t in range(out.shape[0]):
            for s in range(top):
                out[t] += weights[t, s] * (down[int(chosen[t, s])].float() @ hidden[t * top + s].float())

    def sample(self, logits, temperature, uniform, out):
        for row in range(logits.shape[0]):
            temp = float(temperature[row])
            if not temp > 0.0:
                out[row] = int(torch.argmax(logits[row]))
                continue
            weights = torch.exp((logits[row] - logits[row].max()) / temp)
            running = torch.cumsum(weights.double(), dim=0)
            target = float(uniform[row]) * float(running[-1])
            index = int(torch.searchsorted(running, torch.tensor(target, dtype=torch.float64), right=True))
            out[row] = min(index, logits.shape[1] - 1)


class ChunkedMemoryOps(TorchOps):
    """The twins, with the matrix memory in its chunked form where a step brings ``chunked_from`` tokens more than it has
    rows: a row's tokens in chunks of ``chunk`` from its first token of the step; with ``L_t`` the sum of ``log keep`` from
    the chunk's first token to ``t``, the read-outs are ``(Q K^T * W) V + e^(L_t) q_t S_0`` with
    ``W[t, j] = e^(L_t - L_j) take_j`` for ``j <= t``, and the state behind the chunk is
    ``e^(L_last) S_0 + sum_j e^(L_last - L_j) take_j k_j v_j^T``; a column of ones behind the values carries the normaliser."""

    def __init__(self, chunk=64, chunked_from=64):
        super().__init__()
        self.chunk, self.chunked_from, self.chunked_steps = int(chunk), int(chunked_from), 0

    def matrix_memory_chunks(self, n_tokens, rows):
        return n_tokens // self.chunk + rows if n_tokens - rows >= self.chunked_from else 0

    def matrix_memory(self, q, k, v, gates, cap, q_scale, state, state_slots, row_start, row_len, row_ctx, out, below, coefficients,
                      heads, dim, value_dim, run=None, sums=None):
        if run is None:
            assert sums is None
            return super().matrix_memory(q, k, v, gates, cap, q_scale, state, state_slots, row_start, row_len, row_ctx, out, below, coefficients,
                                         heads, dim, value_dim)
        n_tokens = out.shape[0]
        assert tuple(run.shape) == (n_tokens, heads) and run.dtype == torch.float64
        assert tuple(sums.shape[1:]) == (heads, dim, value_dim + 1) and sums.shape[0] >= n_tokens // self.chunk + len(row_len)
        self.chunked_steps += 1
        matrix_size, normaliser_size = heads * dim * value_dim, heads * dim
        log_in = cap * torch.tanh(gates[:, :heads].float() / cap)
        log_forget = torch.nn.functional.logsigmoid(cap * torch.tanh(gates[:, heads:].float() / cap))
        item = 0
        for row in range(len(row_len)):
            start, count, end = int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            if count <= 0:
                continue
            slot = int(state_slots[row])
            kept = state[slot].clone()
            if end - count == 0:
                kept.zero_()
            both = torch.cat([kept[:matrix_size].view(heads, dim, value_dim),
                              kept[matrix_size:matrix_size + normaliser_size].view(heads, dim, 1)], dim=-1)       # [h, d, v + 1]
            top = kept[matrix_size + normaliser_size:matrix_size + normaliser_size + heads].clone()
            for first in range(start, start + count, self.chunk):
                tokens = slice(first, min(first + self.chunk, start + count))
                size = tokens.stop - tokens.start
                log_keep, take = torch.empty(size, heads), torch.empty(size, heads)
                for t in range(size):                                       # the walk of the maximum, token by token
                    new_top = torch.maximum(log_forget[first + t] + top, log_in[first + t])
                    log_keep[t], take[t] = (log_forget[first + t] + top) - new_top, torch.exp(log_in[first + t] - new_top)
                    below[first + t, :, 1] = torch.exp(-new_top)
                    top = new_top
                sums_of_logs = torch.cumsum(log_keep.double(), dim=0)                                  # L [C, h]
                run[tokens] = sums_of_logs
                coefficients[tokens, :, 0], coefficients[tokens, :, 1] = torch.exp(log_keep), take
                queries = q[tokens].float().view(size, heads, dim) * q_scale
                keys = k[tokens].float().view(size, heads, dim)
                values = torch.cat([v[tokens].float().view(size, heads, value_dim), torch.ones(size, heads, 1)], dim=-1)
                behind = torch.tril(torch.ones(size, size, dtype=torch.bool))[:, :, None]                # j <= t
                apart = torch.where(behind, sums_of_logs[:, None, :] - sums_of_logs[None, :, :], torch.tensor(-float("inf"), dtype=torch.float64))
                weights = torch.exp(apart.float()) * take[None, :, :]                                    # [t, j, h]
                scores = torch.einsum("thd,jhd->tjh", queries, keys) * weights
                sums[item] = both                                           # the state in front of the chunk
                read = torch.einsum("tjh,jhv->thv", scores, values) \
                    + torch.exp(sums_of_logs.float())[:, :, None] * torch.einsum("thd,hdv->thv", queries, both)
                out[tokens] = read[..., :value_dim].reshape(size, -1)
                below[tokens, :, 0] = read[..., value_dim]
                to_last = torch.exp((sums_of_logs[-1][None, :] - sums_of_logs).float()) * take                           # [j, h]
                both = torch.exp(sums_of_logs[-1].float())[:, None, None] * both + torch.einsum("jh,jhd,jhv->hdv", to_last, keys, values)
                item += 1
            state[slot, :matrix_size] = both[..., :value_dim].reshape(-1)
            state[slot, matrix_size:matrix_size + normaliser_size] = both[..., value_dim].reshape(-1)
            state[slot, matrix_size + normaliser_size:matrix_size + normaliser_size + heads] = top
