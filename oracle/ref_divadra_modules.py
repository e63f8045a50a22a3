"""Oracle (test infrastructure): torch stand-ins for the layers Divadra is built from (hashed bigram embedding, the
two-norm stream boundary, squared ReLU, causal convolutions with carried inputs, token-shift blends, the decayed memory
with a bonus, the state-space scan, the grouped norm, chunked sigmoid attention over the paged cache, table-routed
experts), with the same constructors and the same cache / state layouts as the HIP-backed modules.  They let the whole
engine run without a GPU and give GPU tests an eager reference per layer.  Device-agnostic, slow, written from the
layer interfaces; the product model never imports it."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .ref_benarax_modules import CausalConvAdd, _ctx, _unit_rms  # noqa: F401  (the same input convolution)


def _spans(ctx):
    """(sequence index, slot, first row, rows, position of the first row) for every sequence with rows in the step."""
    cu_q, cu_k = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist()
    slots = ctx.state_slots.tolist() if ctx.state_slots is not None else [None] * (len(cu_q) - 1)
    for b, slot in enumerate(slots):
        nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
        if nq > 0:
            yield b, slot, cu_q[b], nq, nk - nq


class HashedBigramEmbedding(nn.Module):
    def __init__(self, vocab, width, buckets, mul_prev, mul_cur, eps, dtype=None, device=None, normed=True):
        super().__init__()
        self.buckets, self.mul_prev, self.mul_cur, self.eps = int(buckets), int(mul_prev), int(mul_cur), float(eps)
        self.weight = nn.Parameter(torch.zeros(vocab, width, dtype=dtype, device=device))
        self.bigram = nn.Parameter(torch.zeros(buckets + 1, width, dtype=dtype, device=device)) if buckets else None
        self.norm = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device)) if normed else None

    def forward(self, ids, positions, prev_state):
        x = self.weight[ids].float()
        if self.bigram is not None:
            rows = torch.empty_like(ids)
            for b, slot, r0, nq, start in _spans(_ctx()):
                prev = torch.cat([prev_state[slot].view(1), ids[r0:r0 + nq - 1]])
                rows[r0:r0 + nq] = (prev * self.mul_prev + ids[r0:r0 + nq] * self.mul_cur) % self.buckets
                if start == 0:
                    rows[r0] = self.buckets
                prev_state[slot] = ids[r0 + nq - 1]
            x = x + self.bigram[rows].float()
        return _unit_rms(x, self.eps) * self.norm if self.norm is not None else x


def stream_boundary_pair(x, adds=(), parts=None, parts_scale=1.0, normed=(), normed_mult=1.0, norms=(), eps=1e-5,
                         out_dtype=None, want_f32=True):
    for a in adds:
        x += a.float()
    if parts is not None:
        x += parts_scale * parts.float().sum(1)
    if normed:
        y = torch.zeros_like(x)
        for n, w in normed:
            y = y + _unit_rms(n.float(), eps) * w
        x += normed_mult * y
    if not norms:
        return None, None
    u = _unit_rms(x, eps)
    h32 = torch.cat([u * w for w in norms], dim=1) if want_f32 else None
    return h32, ((u * norms[0]).to(out_dtype) if out_dtype is not None else None)


class ReluSquared(nn.Module):
    def forward(self, x):
        return (torch.relu(x.float()) ** 2).to(x.dtype)


class TokenShiftMix(nn.Module):
    def __init__(self, n_mix, channels, device=None):
        super().__init__()
        self.mu = nn.Parameter(torch.zeros(n_mix, channels, dtype=torch.float32, device=device))

    def forward(self, h, state):
        out = torch.empty((self.mu.shape[0],) + tuple(h.shape), dtype=h.dtype, device=h.device)
        for b, slot, r0, nq, start in _spans(_ctx()):
            cur = h[r0:r0 + nq].float()
            first = state[slot].float() if start > 0 else torch.zeros_like(cur[0])
            prev = torch.cat([first[None], cur[:-1]], dim=0)
            out[:, r0:r0 + nq] = (cur[None] + (prev - cur)[None] * self.mu[:, None, :]).to(h.dtype)
            state[slot] = h[r0 + nq - 1]
        return out


class DecayMemory(nn.Module):
    def __init__(self, num_heads, key_dim, value_dim, eps, device=None):
        super().__init__()
        self.H, self.Dk, self.Dv, self.eps = num_heads, key_dim, value_dim, eps
        f32 = dict(dtype=torch.float32, device=device)
        self.w_bias = nn.Parameter(torch.zeros(num_heads * key_dim, **f32))
        self.bonus = nn.Parameter(torch.zeros(num_heads, key_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(num_heads * value_dim, **f32))

    def forward(self, r, k, v, w_raw, gate_raw, state):
        T, H, Dk, Dv = r.shape[0], self.H, self.Dk, self.Dv
        r, k, v = r.float(), k.float(), v.float()
        w = torch.exp(-torch.exp(w_raw.float() + self.w_bias)).view(T, H, Dk)
        out = torch.zeros(T, H, Dv, dtype=torch.float32, device=r.device)
        for b, slot, r0, nq, start in _spans(_ctx()):
            S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
            for t in range(r0, r0 + nq):
                kv = k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S + self.bonus[:, :, None] * kv, r[t])
                S = w[t][:, :, None] * S + kv
            state[slot] = S
        out = _unit_rms(out, self.eps).reshape(T, H * Dv) * self.norm_weight * F.silu(gate_raw.float())
        return out.to(gate_raw.dtype)


class ConvBiasSilu(nn.Module):
    def __init__(self, channels, taps, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(channels, dtype=torch.float32, device=device))

    def forward(self, x, conv_state):
        keep = self.taps - 1
        y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        for b, slot, r0, nq, start in _spans(_ctx()):
            past = conv_state[slot].float() if start > 0 else torch.zeros(keep, x.shape[1], device=x.device)
            if 0 < start < keep:
                past = past.clone()
                past[:keep - start] = 0
            seq = torch.cat([past, x[r0:r0 + nq].float()], dim=0)
            acc = self.bias.expand(nq, -1).clone()
            for j in range(self.taps):
                acc += seq[j:j + nq] * self.weight[:, j]
            y[r0:r0 + nq] = F.silu(acc).to(x.dtype)
            conv_state[slot] = seq[seq.shape[0] - keep:].to(conv_state.dtype)
        return y


class StateSpaceScan(nn.Module):
    def __init__(self, num_heads, groups, state_dim, head_dim, device=None):
        super().__init__()
        self.H, self.G, self.N, self.P = num_heads, groups, state_dim, head_dim
        f32 = dict(dtype=torch.float32, device=device)
        self.dt_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.A_log = nn.Parameter(torch.zeros(num_heads, **f32))
        self.D = nn.Parameter(torch.zeros(num_heads, **f32))

    def forward(self, x, B, C, dt_raw, z, state):
        T, H, per = x.shape[0], self.H, self.H // self.G
        x, B, C = x.float(), B.float(), C.float()
        dt = F.softplus(dt_raw.float() + self.dt_bias)
        decay = torch.exp(-torch.exp(self.A_log) * dt)
        y = torch.zeros(T, H, self.P, dtype=torch.float32, device=x.device)
        for b, slot, r0, nq, start in _spans(_ctx()):
            S = state[slot].clone() if start > 0 else torch.zeros_like(state[slot])
            for t in range(r0, r0 + nq):
                Bh, Ch = B[t].repeat_interleave(per, dim=0), C[t].repeat_interleave(per, dim=0)
                S = decay[t][:, None, None] * S + (dt[t][:, None] * Bh)[:, :, None] * x[t][:, None, :]
                y[t] = torch.einsum("hnp,hn->hp", S, Ch) + self.D[:, None] * x[t]
            state[slot] = S
        return y.reshape(T, H * self.P) * F.silu(z.float())


def group_rms_norm(x, weight, groups, eps, out_dtype):
    T, C = x.shape
    return (_unit_rms(x.float().view(T, groups, C // groups), eps).reshape(T, C) * weight).to(out_dtype)


def _freqs(dims, base):
    return torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float32)


def _turn(x, positions, freq, dims, sign=1.0):
    half = dims // 2
    ang = positions.float()[:, None] * freq[None, :] * sign
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x = x.float()
    out = x.clone()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half], out[..., half:dims] = a * c - b * s, b * c + a * s
    return out


class ChunkSigmoidAttention(nn.Module):
    def __init__(self, num_heads, num_kv_heads, head_dim, v_head_dim, scale, chunk, rot_dims, rot_base, eps, device=None):
        super().__init__()
        self.H, self.G, self.D, self.Dv = num_heads, num_kv_heads, head_dim, v_head_dim
        self.scale, self.chunk, self.rot_dims, self.eps = float(scale), int(chunk), int(rot_dims), float(eps)
        f32 = dict(dtype=torch.float32, device=device)
        self.q_norm = nn.Parameter(torch.ones(num_heads * head_dim, **f32))
        self.k_norm = nn.Parameter(torch.ones(num_kv_heads * head_dim, **f32))
        self.head_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.register_buffer("freq", _freqs(rot_dims, rot_base).to(device) if rot_dims else None, persistent=False)
        self.register_buffer("value_freq", _freqs(v_head_dim, rot_base).to(device), persistent=False)

    def forward(self, q, k, v, positions, k_cache, v_cache):
        ctx = _ctx()
        dt, T, H, G, D, Dv = q.dtype, q.shape[0], self.H, self.G, self.D, self.Dv
        qn = (_unit_rms(q.reshape(T, H * D), self.eps) * self.q_norm).view(T, H, D)
        kn = (_unit_rms(k.reshape(T, G * D), self.eps) * self.k_norm).view(T, G, D)
        if self.rot_dims:
            qn, kn = _turn(qn, positions, self.freq, self.rot_dims), _turn(kn, positions, self.freq, self.rot_dims)
        qn, kn = qn.to(dt), kn.to(dt)
        vr = _turn(v, positions, self.value_freq, Dv).to(dt)
        bs = k_cache.shape[1]
        slots = ctx.slot_mapping.long()
        k_cache.view(-1, G, D)[slots] = kn
        v_cache.view(-1, G, Dv)[slots] = vr
        cu_q, cu_k = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist()
        out = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
        for b in range(len(cu_q) - 1):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            pos_k = torch.arange(nk, device=q.device)
            rows = ctx.block_tables[b].long()[pos_k // bs] * bs + pos_k % bs
            kk, vv = k_cache.view(-1, G, D)[rows].float(), v_cache.view(-1, G, Dv)[rows].float()
            pos_q = nk - nq + torch.arange(nq, device=q.device)
            vis = pos_k[None, :] <= pos_q[:, None]
            if self.chunk:
                vis = vis & ((pos_k[None, :] // self.chunk) == (pos_q[:, None] // self.chunk))
            qq = qn[cu_q[b]:cu_q[b + 1]].float()
            for h in range(H):
                g = h // (H // G)
                a = torch.sigmoid(qq[:, h] @ kk[:, g].t() * self.scale + self.head_bias[h]) * vis
                out[cu_q[b]:cu_q[b + 1], h] = a @ vv[:, g]
        out = _turn(out, positions, self.value_freq, Dv, sign=-1.0)
        return out.reshape(T, H * Dv).to(dt)


class TableExperts(nn.Module):
    def __init__(self, top):
        super().__init__()
        self.top = int(top)

    def forward(self, h, table, token_ids, gate_up, down):
        T, ff, dt = h.shape[0], gate_up.shape[1] // 2, h.dtype
        idx = table[token_ids].long()
        out = torch.zeros(T, self.top, down.shape[1], dtype=torch.float32, device=h.device)
        for e in idx.unique().tolist():
            t, j = (idx == e).nonzero(as_tuple=True)
            gu = F.linear(h[t], gate_up[e]).float()
            y = (F.silu(gu[:, :ff]) * gu[:, ff:]).to(dt)
            out[t, j] = F.linear(y, down[e]).float()
        return out
