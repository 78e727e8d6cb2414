"""Plain PyTorch references of every kernel the engine calls, one function per kernel.

They take the same arguments as the HIP wrappers in ``velox_amd.kernels`` and work on the
same memory layouts (paged keys ``[pages, kv_heads, page, d]``, paged values
``[pages, kv_heads, d, page]``), so that (1) each HIP kernel is compared with its reference
alone, at sizes of the test's choosing, and (2) the host side of the engine (batching,
cache manager, scheduler) can be exercised on a CPU by handing ``TorchOps`` to it.  The
product never loads this file.
"""
from __future__ import annotations

import numpy as np
import torch


# ----------------------------------------------------------------------------------------
# counter-based generator (Philox 4x32, 10 rounds), as the sampling kernel uses it
# ----------------------------------------------------------------------------------------
_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)


def philox4x32(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """``counter`` uint32 [..., 4], ``key`` uint32 [..., 2] -> uint32 [..., 4]."""
    c = [counter[..., i].astype(np.uint32) for i in range(4)]
    k0 = key[..., 0].astype(np.uint32)
    k1 = key[..., 1].astype(np.uint32)
    for _ in range(10):
        p0 = _M0 * c[0].astype(np.uint64)
        p1 = _M1 * c[2].astype(np.uint64)
        hi0, lo0 = (p0 >> np.uint64(32)).astype(np.uint32), p0.astype(np.uint32)
        hi1, lo1 = (p1 >> np.uint64(32)).astype(np.uint32), p1.astype(np.uint32)
        c = [hi1 ^ c[1] ^ k0, lo1, hi0 ^ c[3] ^ k1, lo0]
        k0 = (k0 + _W0).astype(np.uint32)
        k1 = (k1 + _W1).astype(np.uint32)
    return np.stack(c, axis=-1)


def exponential_noise(vocab: int, seed_lo: int, seed_hi: int, counter: int) -> np.ndarray:
    """Exp(1) noise of one row: element i uses lane i % 4 of block i // 4; u = (bits >> 8 + 0.5) / 2^24."""
    blocks = (vocab + 3) // 4
    ctr = np.zeros((blocks, 4), dtype=np.uint32)
    ctr[:, 0] = np.arange(blocks, dtype=np.uint32)
    ctr[:, 1] = np.uint32(counter)
    key = np.zeros((blocks, 2), dtype=np.uint32)
    key[:, 0] = np.uint32(seed_lo)
    key[:, 1] = np.uint32(seed_hi)
    bits = philox4x32(ctr, key).reshape(-1)[:vocab]
    u = ((bits >> np.uint32(8)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 16777216.0)
    return np.maximum(-np.log(u), np.float32(1e-10)).astype(np.float32)


class TorchOps:
    """The kernels' arithmetic in plain PyTorch, on whatever device the tensors live."""

    name = "torch-reference"

    def prepare(self, model, dtype) -> None:
        pass

    def materialize(self, x):
        return x

    def qkv_rope_write(self, x, weight, bias, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=True):
        qkv = self.linear(x, weight, None, x.dtype)
        self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=write_kv, bias=bias)
        return qkv

    # -- embedding and norms ------------------------------------------------------------
    def place_tokens(self, ids, dest, source, tokens, count):
        ids[dest[:count].long()] = tokens[source[:count].long()]

    def embed(self, token_ids, table, scale=1.0, copies=1):
        out = table[token_ids.long()].float()
        out = out * scale if scale != 1.0 else out
        return out.repeat(1, copies) if copies != 1 else out

    def embed_bigram(self, token_ids, table, bigram, scale, buckets, mul_prev, mul_cur, positions, cu_q, slots, state, max_q_len=None):
        """Row of the table times ``scale`` plus the row of ``bigram`` that (previous token, token) hash to; position 0 reads
        row ``buckets``; a portion's first token takes the previous one from ``state`` [slots, 1], which then takes the
        portion's last token."""
        ids = token_ids.long()
        previous = torch.roll(ids, 1)
        starts, ends = cu_q[:-1].long(), cu_q[1:].long()
        previous[starts] = state[slots.long(), 0].long()
        rows = (previous * mul_prev + ids * mul_cur) % buckets
        rows = torch.where(positions.long() == 0, torch.full_like(rows, buckets), rows)
        state[slots.long(), 0] = ids[ends - 1].to(state.dtype)
        return table[ids].float() * scale + bigram[rows].float()

    def add_dynamic_tanh(self, residual, delta, weight, bias, alpha, out_dtype, rows=None):
        """``residual += delta`` (float32; with ``rows`` nothing is changed and only those rows are worked), then
        ``tanh(alpha x) * weight + bias``."""
        delta = self._one_delta(delta)
        if delta is not None and delta.dim() == 3:
            delta = delta.float().sum(0)
        if rows is None:
            if delta is not None:
                residual += delta.float()
            x = residual
        else:
            x = residual[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].float()
        return (torch.tanh(alpha.float() * x) * weight.float() + bias.float()).to(out_dtype)

    def scale_(self, x, factor):
        return x.mul_(factor)

    def activation(self, x, kind):
        if kind != "relu2":
            raise ValueError(kind)
        return torch.relu(x.float()).square().to(x.dtype)

    def linear_act(self, x, weight, out_dtype, kind):
        """``act(x W^T)``: the activation on the float32 sums, one rounding."""
        if kind != "relu2":
            raise ValueError(kind)
        return torch.relu(x.float() @ weight.float().T).square().to(out_dtype)

    def stream_norm(self, residual, terms, scales, mix, out_weights, in_weights, weight, eps, streams, center, out_dtype, rows=None):
        """``residual`` float32 [T, S * H].  With terms: ``x_t <- sum_s mix[s, t] x_s + out[t] * y`` where ``y = sum_i scales[i]
        terms[i]`` (mix None: identity, out None: ones), in place unless ``rows`` is given.  Returns the norm of
        ``u = sum_s in[s] x_s`` (in None: ones) times ``weight``, for all rows or for ``rows``."""
        t = residual.shape[0]
        h = residual.shape[1] // streams
        select = slice(None) if rows is None else rows.long()
        x = residual.view(t, streams, h)[select]
        if len(terms):
            y = sum(float(s) * term[select].float() for s, term in zip(scales, terms))
            mixed = x if mix is None else torch.einsum("st,nsh->nth", mix.float(), x)
            weights = torch.ones(streams, device=x.device) if out_weights is None else out_weights.float()
            x = mixed + weights[None, :, None] * y[:, None, :]
            if rows is None:
                residual.view(t, streams, h).copy_(x)
        u = x.sum(1) if in_weights is None else torch.einsum("s,nsh->nh", in_weights.float(), x)
        if center:
            u = u - u.mean(-1, keepdim=True)
        var = (u * u).mean(-1, keepdim=True)
        return (u / torch.sqrt(var + eps) * weight.float()).to(out_dtype)

    def gated_act_mul(self, gate_up, activation):
        inter = gate_up.shape[-1] // 2
        gate, up = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        if activation == "gelu_tanh":
            act = 0.5 * gate * (1.0 + torch.tanh(0.7978845608028654 * (gate + 0.044715 * gate * gate * gate)))
        elif activation == "silu":
            act = gate * torch.sigmoid(gate)
        else:
            raise ValueError(activation)
        return (act * up).to(gate_up.dtype)

    # -- short convolution, recurrences -------------------------------------------------------
    def short_conv(self, x, channels, weight, tail, slots, cu_q, max_q_len, activation="none", update_state=True):
        """``x`` [T, >= channels]: the first ``channels`` columns pass ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)`` per sequence,
        the inputs before a portion's start come from ``tail[slot]`` ([taps - 1, channels], oldest first), which is then
        brought up to date.  Returns [T, channels] in x's dtype."""
        taps = weight.shape[1]
        out = torch.empty((x.shape[0], channels), dtype=x.dtype, device=x.device)
        bounds = cu_q.tolist()
        for b, slot in enumerate(slots.tolist()):
            lo, hi = bounds[b], bounds[b + 1]
            u = x[lo:hi, :channels].float()
            if taps > 1:
                before = tail[slot].float() if tail is not None else torch.zeros((taps - 1, channels), device=x.device)
                u = torch.cat([before, u], 0)
            y = sum(weight[:, j].float() * u[j:j + hi - lo] for j in range(taps))
            if activation == "silu":
                y = y * torch.sigmoid(y)
            out[lo:hi] = y.to(x.dtype)
            if taps > 1 and tail is not None and update_state:
                tail[slot] = u[u.shape[0] - (taps - 1):].to(tail.dtype)
        return out

    def rotate_pad_write(self, qkv, num_heads, num_kv_heads, dim, vdim, cached_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=True,
                         interleaved=False):
        """Rotates the first ``2 * cos.shape[1]`` channels of every q and k head (halves layout, or pairs (2i, 2i + 1)), writes k and v into the
        pages at ``cached_dim`` channels a head (zeros in the padding) and returns q as [T, heads * cached_dim]."""
        t = qkv.shape[0]
        q_size, k_size = num_heads * dim, num_kv_heads * dim
        q = qkv[:, :q_size].float().view(t, num_heads, dim)
        k = qkv[:, q_size:q_size + k_size].float().view(t, num_kv_heads, dim)
        v = qkv[:, q_size + k_size:].float().view(t, num_kv_heads, vdim)
        if cos is not None:
            half = cos.shape[1]
            c, s_ = cos[positions.long()][:, None, :], sin[positions.long()][:, None, :]

            def rotate(x):
                if interleaved:
                    return self._rotate(x, c, s_, True)
                a, b = x[..., :half], x[..., half:2 * half]
                return torch.cat([a * c - b * s_, b * c + a * s_, x[..., 2 * half:]], -1)

            q, k = rotate(q), rotate(k)
        out = torch.zeros((t, num_heads, cached_dim), dtype=qkv.dtype, device=qkv.device)
        out[:, :, :dim] = q.to(qkv.dtype)
        if write_kv:
            page, offset = (slot_mapping // block_size).long(), (slot_mapping % block_size).long()
            k_pad = torch.zeros((t, num_kv_heads, cached_dim), dtype=k_cache.dtype, device=qkv.device)
            k_pad[:, :, :dim] = k.to(k_cache.dtype)
            v_pad = torch.zeros((t, num_kv_heads, cached_dim), dtype=v_cache.dtype, device=qkv.device)
            v_pad[:, :, :vdim] = v.to(v_cache.dtype)
            k_cache[page, :, offset, :] = k_pad
            v_cache[page, :, :, offset] = v_pad
        return out.view(t, num_heads * cached_dim)

    def recurrence_prepare(self, qkv, q_at, k_at, kv_heads, dim, unit, q_scale, decay_source, decay_at, heads, decay_columns, rate, bias, sign,
                           beta_source, beta_at):
        """-> qk float32 [T, kv_heads, 2, dim] (q then k of a head), decay float32 [T, decay_columns] =
        ``exp(-rate[h] * softplus(sign * (z + bias)))``, beta float32 [T, heads] = ``sigmoid(b)`` or None."""
        t = qkv.shape[0]
        q = qkv[:, q_at:q_at + kv_heads * dim].float().view(t, kv_heads, dim)
        k = qkv[:, k_at:k_at + kv_heads * dim].float().view(t, kv_heads, dim)
        if unit:
            q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6)
            k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        qk = torch.stack([q * q_scale, k], 2).contiguous()
        z = decay_source[:, decay_at:decay_at + decay_columns].float()
        if bias is not None:
            z = z + bias.float()
        per_head = decay_columns // heads
        decay = torch.exp(-rate.float().repeat_interleave(per_head)[None, :] * torch.nn.functional.softplus(sign * z)).contiguous()
        beta = None
        if beta_source is not None:
            beta = torch.sigmoid(beta_source[:, beta_at:beta_at + heads].float()).contiguous()
        return qk, decay, beta

    def linear_scan(self, qk, v_source, v_at, decay, beta, state, slots, cu_q, max_q_len, heads, kv_heads, dim, vdim, delta):
        """Per sequence and head, token by token from ``state[slot, head]`` ([dim, vdim] float32), which is written back:
        ``S <- g S`` (rows); ``u = beta (v - S^T k)`` (delta) or ``u = v``; ``o = S^T q + (k . q) u``; ``S <- S + k u^T``.
        Returns float32 [T, heads * vdim]."""
        t = qk.shape[0]
        out = torch.empty((t, heads, vdim), dtype=torch.float32, device=qk.device)
        v = v_source[:, v_at:v_at + heads * vdim].float().view(t, heads, vdim)
        g = decay.view(t, heads, -1)
        repeat = heads // kv_heads
        bounds = cu_q.tolist()
        for b, slot in enumerate(slots.tolist()):
            s = state[slot].clone()  # [heads, dim, vdim]
            for i in range(bounds[b], bounds[b + 1]):
                q = qk[i, :, 0].repeat_interleave(repeat, 0)  # [heads, dim]
                k = qk[i, :, 1].repeat_interleave(repeat, 0)
                s = s * g[i][:, :, None]
                u = v[i]
                if delta:
                    u = beta[i][:, None] * (u - torch.einsum("hde,hd->he", s, k))
                out[i] = torch.einsum("hde,hd->he", s, q) + (k * q).sum(-1, keepdim=True) * u
                s = s + k[:, :, None] * u[:, None, :]
            state[slot] = s
        return out.view(t, heads * vdim)

    def gated_head_norm(self, read, weight, eps, gate_source, gate_at, gate_kind, heads, vdim, out_dtype):
        t = read.shape[0]
        o = read.view(t, heads, vdim)
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * weight.float()
        gate = gate_source[:, gate_at:gate_at + heads * vdim].float().view(t, heads, vdim)
        gate = gate * torch.sigmoid(gate) if gate_kind == "silu" else torch.sigmoid(gate)
        return (o * gate).view(t, heads * vdim).to(out_dtype)

    @staticmethod
    def _one_delta(delta):
        from velox_amd.parts.base import SumOf

        if isinstance(delta, SumOf):
            first = delta.first.float().sum(0) if delta.first.dim() == 3 else delta.first.float()
            return first + delta.second.float()
        return delta

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype):
        delta = self._one_delta(delta)
        if delta is not None and delta.dim() == 3:
            delta = delta.float().sum(0)
        if delta is not None:
            residual += delta.float()
        var = (residual * residual).sum(-1, keepdim=True) / residual.shape[-1]
        return (residual * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps, out_dtype):
        delta = self._one_delta(delta)
        if delta is not None and delta.dim() == 3:
            delta = delta.float().sum(0)
        x = residual[rows.long()]
        if delta is not None:
            x = x + delta[rows.long()].float()
        var = (x * x).sum(-1, keepdim=True) / x.shape[-1]
        return (x * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)

    def add_sinusoid(self, hidden, positions, frequencies):
        """hidden[t, 2i] += sin(p_t f_i), hidden[t, 2i + 1] += cos(p_t f_i), in place."""
        angle = positions.double()[:, None] * frequencies.double()[None, :]
        width = hidden.shape[1]
        hidden[:, 0::2] += torch.sin(angle).float()[:, : (width + 1) // 2]
        hidden[:, 1::2] += torch.cos(angle).float()[:, : width // 2]
        return hidden

    def add_cast(self, residual, delta, out_dtype):
        if delta is not None:
            residual += delta.float()
        return residual if out_dtype == torch.float32 else residual.to(out_dtype)

    def norm_add(self, residual, delta, weight, eps, mult, out_dtype):
        y = delta.float().sum(0) if delta.dim() == 3 else delta.float()
        var = (y * y).sum(-1, keepdim=True) / y.shape[-1]
        residual += mult * (y / torch.sqrt(var + eps) * weight.float())
        return residual if out_dtype == torch.float32 else residual.to(out_dtype)

    def qk_norm_write(self, qkv, num_heads, num_kv_heads, dim, vdim, cached_dim, q_norm, k_norm, whole, eps, q_temp, positions, first_values,
                      mix_weight, slot_mapping, k_cache, v_cache, block_size, write_kv=True):
        t = qkv.shape[0]
        q_size, k_size, v_size = num_heads * dim, num_kv_heads * dim, num_kv_heads * vdim
        wide = qkv.float()
        q, k, v = wide[:, :q_size], wide[:, q_size:q_size + k_size], wide[:, q_size + k_size:q_size + k_size + v_size]

        def unit(x):
            return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)

        if whole:
            q = (unit(q) * q_norm.float()).view(t, num_heads, dim)
            k = (unit(k) * k_norm.float()).view(t, num_kv_heads, dim)
        else:
            q = unit(q.reshape(t, num_heads, dim)) * q_norm.float()
            k = unit(k.reshape(t, num_kv_heads, dim)) * k_norm.float()
        if q_temp is not None:
            coef, every = q_temp
            steps = torch.div(positions.long() + 1, int(every), rounding_mode="floor") + 1
            q = q * (1.0 + coef * torch.log(steps.float()))[:, None, None]
        if first_values is not None:
            source, offset = first_values
            lam = mix_weight.float().reshape(())
            v = (1.0 - lam) * v + lam * source[:, offset:offset + v_size].float()
        out = torch.zeros((t, num_heads, cached_dim), dtype=qkv.dtype, device=qkv.device)
        out[:, :, :dim] = q.to(qkv.dtype)
        if write_kv:
            pages = slot_mapping.long() // block_size
            offsets = slot_mapping.long() % block_size
            keys = torch.zeros((t, num_kv_heads, cached_dim), dtype=k_cache.dtype, device=qkv.device)
            keys[:, :, :dim] = k.to(k_cache.dtype)
            values = torch.zeros((t, num_kv_heads, cached_dim), dtype=v_cache.dtype, device=qkv.device)
            values[:, :, :vdim] = v.reshape(t, num_kv_heads, vdim).to(v_cache.dtype)
            k_cache[pages, :, offsets, :] = keys
            v_cache[pages, :, :, offsets] = values
        return out.view(t, num_heads * cached_dim)

    # -- matrix products ----------------------------------------------------------------
    def linear(self, x, weight, bias, out_dtype, partials_ok=False, residual_norm=None):
        out = x.float() @ weight.float().T
        if bias is not None:
            out = out + bias.float()
        return out.to(out_dtype)

    def linear_silu_mul(self, x, gate_up_weight, out_dtype, **_):
        return self.silu_mul(self.linear(x, gate_up_weight, None, out_dtype))

    def silu_mul(self, gate_up):
        inter = gate_up.shape[-1] // 2
        gate = gate_up[:, :inter].float()
        up = gate_up[:, inter:].float()
        return (gate * torch.sigmoid(gate) * up).to(gate_up.dtype)

    # -- rotary + cache write -----------------------------------------------------------
    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=True, bias=None):
        t = qkv.shape[0]
        q_size, kv_size = num_heads * head_dim, num_kv_heads * head_dim
        wide = qkv.float()
        if bias is not None:
            wide = wide + bias
        q = wide[:, :q_size].reshape(t, num_heads, head_dim).clone()
        k = wide[:, q_size:q_size + kv_size].reshape(t, num_kv_heads, head_dim).clone()
        v = wide[:, q_size + kv_size:].reshape(t, num_kv_heads, head_dim)
        if cos is not None:
            half = cos.shape[1]
            c = cos[positions.long()].unsqueeze(1)
            s = sin[positions.long()].unsqueeze(1)
            for x in (q, k):
                lo = x[..., :half].clone()
                hi = x[..., half:2 * half].clone()
                x[..., :half] = lo * c - hi * s
                x[..., half:2 * half] = lo * s + hi * c
        # one rounding, at the store; only the rotated queries go back into qkv
        qkv[:, :q_size] = q.reshape(t, q_size).to(qkv.dtype)
        if write_kv:
            pages = (slot_mapping.long() // block_size)
            offsets = (slot_mapping.long() % block_size)
            k_cache[pages, :, offsets, :] = k.to(k_cache.dtype)
            v_cache[pages, :, :, offsets] = v.to(v_cache.dtype)

    # -- attention over a cached latent ---------------------------------------------------
    @staticmethod
    def _rotate(x, cos, sin, interleaved):
        """``x`` float32 [T, ..., n]; rotates its first 2 * table width channels."""
        half = cos.shape[-1]
        while cos.dim() < x.dim():
            cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
        out = x.clone()
        if interleaved:
            u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
            out[..., 0:2 * half:2] = u * cos - v * sin
            out[..., 1:2 * half:2] = v * cos + u * sin
        else:
            u, v = x[..., :half], x[..., half:2 * half]
            out[..., :half] = u * cos - v * sin
            out[..., half:2 * half] = v * cos + u * sin
        return out

    def latent_rotate_write(self, projected, num_heads, dim, rot_dim, kv_rank, cached_dim, down_offset, positions, cos, sin, interleaved,
                            norm_weight, eps, slot_mapping, k_cache, v_cache, block_size):
        t = projected.shape[0]
        wide = projected.float()
        c = s = None
        if cos is not None:
            c, s = cos[positions.long()], sin[positions.long()]
        queries = torch.zeros((t, num_heads, cached_dim), dtype=projected.dtype, device=projected.device)
        turned = wide[:, : num_heads * (dim + rot_dim)].view(t, num_heads, dim + rot_dim)[..., dim:]
        if c is not None:
            turned = self._rotate(turned, c, s, interleaved)
        queries[..., kv_rank:kv_rank + rot_dim] = turned.to(projected.dtype)
        if down_offset >= 0:
            latent = wide[:, down_offset:down_offset + kv_rank]
            latent = latent / torch.sqrt((latent * latent).mean(-1, keepdim=True) + eps) * norm_weight.float()
            shared = wide[:, down_offset + kv_rank:down_offset + kv_rank + rot_dim]
            if c is not None:
                shared = self._rotate(shared, c, s, interleaved)
            row = torch.zeros((t, cached_dim), dtype=k_cache.dtype, device=projected.device)
            row[:, :kv_rank] = latent.to(k_cache.dtype)
            row[:, kv_rank:kv_rank + rot_dim] = shared.to(k_cache.dtype)
            pages = slot_mapping.long() // block_size
            offsets = slot_mapping.long() % block_size
            k_cache[pages, 0, offsets, :] = row
            v_cache[pages, 0, :, offsets] = row
        return queries.view(t, num_heads * cached_dim)

    def latent_write(self, projected, rot_dim, kv_rank, cached_dim, down_offset, positions, cos, sin, interleaved, norm_weight, eps, slot_mapping,
                     k_cache, v_cache, block_size, q_latent=None):
        """The cache write of ``latent_rotate_write`` without any queries; ``q_latent = (offset, rank, weight)``: those
        columns come back RMS-normed with the weight, [T, rank]."""
        self.latent_rotate_write(projected, 0, 0, rot_dim, kv_rank, cached_dim, down_offset, positions, cos, sin, interleaved, norm_weight, eps,
                                 slot_mapping, k_cache, v_cache, block_size)
        if q_latent is None:
            return None
        offset, rank, weight = q_latent
        part = projected[:, offset:offset + rank].float()
        return (part / torch.sqrt((part * part).mean(-1, keepdim=True) + eps) * weight.float()).to(projected.dtype)

    def head_linear(self, x, x_head_stride, x_offset, maps, out, out_head_stride, out_offset, gate=None, gate_offset=0, gate_per_head=False):
        groups, n, k = maps.shape
        t = x.shape[0]
        for g in range(groups):
            a = x[:, g * x_head_stride + x_offset:g * x_head_stride + x_offset + k].float()
            y = a @ maps[g].float().T
            if gate is not None and gate_per_head:
                y = y * torch.sigmoid(gate[:, gate_offset + g:gate_offset + g + 1].float())
            elif gate is not None:
                y = y * torch.sigmoid(gate[:, gate_offset + g * n:gate_offset + (g + 1) * n].float())
            out[:, g * out_head_stride + out_offset:g * out_head_stride + out_offset + n] = y.to(out.dtype)
        return out

    # -- routed experts -------------------------------------------------------------------
    def route_top(self, logits, top, score="sigmoid", renormalize=False, correction=None, groups=None, norm_floor=0.0):
        scores = torch.sigmoid(logits.float()) if score == "sigmoid" else torch.softmax(logits.float(), dim=-1)
        ranked = scores + correction.float() if correction is not None else scores  # the correction steers the choice only
        if groups is not None:  # only experts of the best groups can be chosen; a group's score: its two largest choice scores
            count, keep = groups
            per = ranked.shape[-1] // count
            grouped = ranked.view(-1, count, per)
            best = grouped.topk(min(2, per), dim=-1).values.sum(-1).topk(keep, dim=-1).indices
            allowed = torch.zeros((ranked.shape[0], count), dtype=torch.bool, device=ranked.device).scatter_(1, best, True)
            ranked = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(ranked.shape)
        choice = ranked.topk(top, dim=-1).indices
        weight = scores.gather(-1, choice)
        if renormalize:
            weight = weight / (weight.sum(-1, keepdim=True) + norm_floor)
        return choice.to(torch.int32), weight

    def routed_experts(self, x, choice, weight, gate_up_weight, down_weight, num_experts, scale_input, shared, out_dtype, workspace=None,
                       unit=(1.0, float("inf"), 0.0), identity_experts=0, output_norm=None, ungated=None):
        alpha, limit, shift = unit
        t, h = x.shape
        branches = 1 if ungated else 2
        f = gate_up_weight.shape[0] // (branches * num_experts)
        gate_up = gate_up_weight.view(num_experts, branches * f, h).float()
        down = down_weight.view(num_experts, h, f).float()
        out = torch.zeros((t, h), dtype=torch.float32, device=x.device)
        for k in range(choice.shape[1]):  # a token's results are added in the order of its choices
            rows = (choice[:, k] >= num_experts).nonzero().flatten()
            if rows.numel():  # identity experts: the input itself, times the weight
                out[rows] += x[rows].float() * weight[rows, k:k + 1]
            for e in range(num_experts):
                rows = (choice[:, k] == e).nonzero().flatten()
                if not rows.numel():
                    continue
                w = weight[rows, k:k + 1]
                a = (x[rows].float() * w).to(x.dtype).float() if scale_input else x[rows].float()
                both = a @ gate_up[e].T
                if ungated:
                    assert ungated == "relu2"
                    act = torch.relu(both).square().to(x.dtype).float()
                else:
                    gate, up = both[:, :f].clamp(max=limit), both[:, f:].clamp(min=-limit, max=limit)
                    act = (gate * torch.sigmoid(alpha * gate) * (up + shift)).to(x.dtype).float()
                y = act @ down[e].T
                out[rows] += y if scale_input else y * w
        if shared is not None:
            out = out + shared.float()
        if output_norm is not None:  # the sum goes to the norm as it is, in float32
            from velox_amd.parts.base import ResidualCopy

            return ResidualCopy(self.norm_add(output_norm.residual, out, output_norm.weight, output_norm.eps, output_norm.mult, out_dtype))
        return out.to(out_dtype)

    # -- attention over the paged cache -------------------------------------------------
    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_size, block_tables, cu_q, kv_lens, max_q_len, max_kv_len, scale, window, all_decode, workspace, splits=None, decode_prefix=0, portions_max_kv_len=None,
                        distance_bias=None, sinks=None):
        """``distance_bias``: float32 [heads, L]; the score of a key ``n`` behind the query gets column ``min(n, L - 1)``.
        ``sinks``: float32 [heads]; ``exp(sinks[h])`` joins the denominator of every row of head ``h``."""
        t = qkv.shape[0]
        group = num_heads // num_kv_heads
        q_all = qkv[:, : num_heads * head_dim].view(t, num_heads, head_dim)
        out = torch.zeros((t, num_heads, head_dim), dtype=torch.float32, device=qkv.device)
        cu = cu_q.tolist()
        lens = kv_lens.tolist()
        for b in range(len(lens)):
            lo, hi = cu[b], cu[b + 1]
            q_len, kv_len = hi - lo, lens[b]
            ctx = kv_len - q_len
            index = torch.arange(kv_len, device=qkv.device)
            pages = block_tables[b].long()[index // block_size]
            offsets = index % block_size
            keys = k_cache[pages, :, offsets, :].float()  # [kv_len, nkv, d]
            values = v_cache[pages, :, :, offsets].float()  # [kv_len, nkv, d]
            q_pos = ctx + torch.arange(q_len, device=qkv.device)
            keep = q_pos[:, None] >= index[None, :]
            if window is not None:
                keep &= index[None, :] > q_pos[:, None] - window
            for h in range(num_heads):
                kv = h // group
                scores = (q_all[lo:hi, h].float() @ keys[:, kv].T) * scale
                if distance_bias is not None:
                    behind = (q_pos[:, None] - index[None, :]).clamp(min=0, max=distance_bias.shape[1] - 1)
                    scores = scores + distance_bias[h].float()[behind]
                scores = scores.masked_fill(~keep, float("-inf"))
                m = scores.max(-1, keepdim=True).values
                p = torch.exp(scores - m)
                denom = p.sum(-1, keepdim=True)
                if sinks is not None:
                    denom = denom + torch.exp(sinks[h].float() - m)
                p = p.to(qkv.dtype).float()  # the kernel rounds p to the value dtype for the second product
                out[lo:hi, h] = (p @ values[:, kv]) / denom
        return out.to(qkv.dtype).view(t, num_heads * head_dim)

    # -- sampling -----------------------------------------------------------------------
    def argmax(self, logits):
        return logits.argmax(dim=-1).to(torch.int32)

    def sample(self, logits, options, with_filter=True, chunks=None):
        return torch.tensor(
            [self.sample_row(logits[r].cpu().numpy(), options[r].cpu().numpy())[0] for r in range(logits.shape[0])],
            dtype=torch.int32, device=logits.device,
        )

    @staticmethod
    def sample_row(row: np.ndarray, option: np.ndarray):
        """One row of the sampling kernel; returns (token, scores) with -inf for dropped tokens."""
        as_float = option.view(np.float32)
        temperature, top_p = float(as_float[0]), float(as_float[1])
        top_k, seed_lo, seed_hi, counter = int(option[2]), int(option[3]), int(option[4]), int(option[5])
        row = row.astype(np.float32)
        if temperature == 0.0:
            return int(row.argmax()), row
        x = row / np.float32(max(temperature, 1e-5))
        x = x - x.max()
        p = np.exp(x.astype(np.float64))
        p = p / p.sum()
        order = np.argsort(-x, kind="stable")
        keep = np.ones_like(x, dtype=bool)
        sorted_x = x[order]
        sorted_p = p[order]
        exclusive = np.cumsum(sorted_p) - sorted_p
        # tokens of equal value share rank and mass: the first of a run decides for all of it
        first_of_run = np.concatenate([[0], np.flatnonzero(np.diff(sorted_x) != 0) + 1])
        run_id = np.zeros(len(x), dtype=np.int64)
        run_id[first_of_run] = 1
        run_id = np.cumsum(run_id) - 1
        rank = first_of_run[run_id]
        mass = exclusive[first_of_run][run_id]
        keep_sorted = mass < top_p
        if top_k > 0:
            keep_sorted &= rank < top_k
        keep[order] = keep_sorted
        noise = exponential_noise(len(x), seed_lo, seed_hi, counter)
        scores = np.where(keep, x - np.log(noise), -np.inf).astype(np.float32)
        return int(scores.argmax()), scores

    def count_tokens(self, counts_row, tokens):
        ok = (tokens >= 0) & (tokens < counts_row.numel())
        counts_row += torch.bincount(tokens[ok].long(), minlength=counts_row.numel()).to(counts_row.dtype)

    def count_sampled(self, counts, row_of, tokens):
        for r in range(tokens.numel()):
            if int(row_of[r]) >= 0 and 0 <= int(tokens[r]) < counts.shape[1]:
                counts[int(row_of[r]), int(tokens[r])] += 1

    def apply_penalties_from_counts(self, logits, counts, row_of, coeffs):
        for r in range(logits.shape[0]):
            if int(row_of[r]) < 0:
                continue
            repetition, presence, frequency = (float(c) for c in coeffs[r])
            seen = counts[int(row_of[r])]
            ids = torch.nonzero(seen).flatten()
            vals = logits[r, ids] - frequency * seen[ids].float()
            vals = torch.where(vals > 0, vals / repetition, vals * repetition) - presence
            logits[r, ids] = vals

    def apply_penalties(self, logits, tokens, lengths, coeffs):
        """engine/sampler.py:169-189 of the reference: frequency first (times the count), then repetition
        (positive / r, negative * r) and presence, each once per distinct seen token."""
        for r in range(logits.shape[0]):
            seen = tokens[r, : int(lengths[r])].long()
            if seen.numel() == 0:
                continue
            repetition, presence, frequency = (float(c) for c in coeffs[r])
            ids, counts = torch.unique(seen, return_counts=True)
            vals = logits[r, ids] - frequency * counts.float()
            vals = torch.where(vals > 0, vals / repetition, vals * repetition) - presence
            logits[r, ids] = vals
