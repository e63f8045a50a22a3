"""Oracle (test infrastructure): torch stand-ins for the layers Tutedra is built from (un-normed hashed bigram embedding,
the scaled stream boundary, one-plus norms, the polynomial-of-norms activation, the token shift, the exponential-gate
matrix memory, the gated-write recurrence, the plain short convolution, attention whose values are its raw keys, sigmoid
routing over groups, squared-ReLU experts), with the same constructors and the same cache / state layouts as the
HIP-backed modules.  They let the whole engine run without a GPU and give GPU tests an eager reference per layer.
Device-agnostic, slow, written from the layer interfaces; the product model never imports it."""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .ref_benarax_modules import _ctx, _unit_rms
from .ref_divadra_modules import HashedBigramEmbedding, ReluSquared, TokenShiftMix, _spans, _turn  # noqa: F401


def stream_boundary_scaled(x, add=None, gated=None, parts=None, col_scale=None, norm=None, eps=1e-5, out_dtype=None,
                           want_f32=False):
    y = None
    if add is not None:
        y = add.float()
    if gated is not None:
        a2, g = gated
        t = a2.float() * (torch.sigmoid(g.float())[:, None] if g is not None else 1.0)
        y = t if y is None else y + t
    if parts is not None:
        t = parts.float().sum(1)
        y = t if y is None else y + t
    if y is not None:
        x += y * col_scale if col_scale is not None else y
    if norm is None:
        return None, None
    u = _unit_rms(x, eps) * norm
    return (u if want_f32 else None), (u.to(out_dtype) if out_dtype is not None else None)


class OnePlusNorm(nn.Module):
    def __init__(self, width, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(width, dtype=torch.float32, device=device))
        self.register_buffer("applied", torch.ones(width, dtype=torch.float32, device=device), persistent=False)

    def finalize(self):
        self.applied = 1.0 + self.weight.data.float()


class PolyNorm(nn.Module):
    def __init__(self, eps, device=None):
        super().__init__()
        self.eps = float(eps)
        self.coef = nn.Parameter(torch.zeros(4, dtype=torch.float32, device=device))

    def forward(self, z):
        u = z.float()
        a, b, c, e = self.coef.tolist()
        return (a * _unit_rms(u, self.eps) + b * _unit_rms(u * u, self.eps) + c * _unit_rms(u * u * u, self.eps) + e).to(z.dtype)


class MatrixLSTMMemory(nn.Module):
    def __init__(self, num_heads, key_dim, value_dim, gate_cap, eps, device=None):
        super().__init__()
        self.H, self.Dk, self.Dv = num_heads, key_dim, value_dim
        self.cap, self.eps, self.q_scale = float(gate_cap), float(eps), float(key_dim) ** -0.5
        f32 = dict(dtype=torch.float32, device=device)
        self.i_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.f_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.norm_weight = nn.Parameter(torch.ones(num_heads * value_dim, **f32))

    def state_shapes(self):
        H, Dk, Dv = self.H, self.Dk, self.Dv
        return {"state": ((H, Dk, Dv), torch.float32), "normaliser": ((H, Dk), torch.float32), "maximum": ((H,), torch.float32)}

    def forward(self, q, k, v, gates_pre, gate_raw, cache):
        T, H = q.shape[0], self.H
        q, k, v = q.float() * self.q_scale, k.float(), v.float()
        gi = self.cap * torch.tanh((gates_pre[:, :H] + self.i_bias) / self.cap)
        gf = F.logsigmoid(self.cap * torch.tanh((gates_pre[:, H:] + self.f_bias) / self.cap))
        out = torch.zeros(T, H, self.Dv, dtype=torch.float32, device=q.device)
        S_all, n_all, m_all = cache["state"], cache["normaliser"], cache["maximum"]
        for b, slot, r0, nq, start in _spans(_ctx()):
            if start > 0:
                S, n, m = S_all[slot].clone(), n_all[slot].clone(), m_all[slot].clone()
            else:
                S, n, m = torch.zeros_like(S_all[slot]), torch.zeros_like(n_all[slot]), torch.zeros_like(m_all[slot])
            for t in range(r0, r0 + nq):
                m_new = torch.maximum(gf[t] + m, gi[t])
                keep, write = torch.exp(gf[t] + m - m_new), torch.exp(gi[t] - m_new)
                S = keep[:, None, None] * S + write[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
                n = keep[:, None] * n + write[:, None] * k[t]
                m = m_new
                den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
                out[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den[:, None]
            S_all[slot], n_all[slot], m_all[slot] = S, n, m
        out = _unit_rms(out, self.eps).reshape(T, H * self.Dv) * self.norm_weight * torch.sigmoid(gate_raw.float())
        return out.to(gate_raw.dtype)


class GatedWriteMemory(nn.Module):
    def __init__(self, num_heads, key_dim, value_dim, eps, device=None):
        super().__init__()
        self.H, self.Dk, self.Dv, self.eps = num_heads, key_dim, value_dim, float(eps)
        f32 = dict(dtype=torch.float32, device=device)
        self.f_bias = nn.Parameter(torch.zeros(num_heads * key_dim, **f32))
        self.lower = nn.Parameter(torch.zeros(num_heads * key_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(value_dim, **f32))

    def state_shapes(self):
        return {"state": ((self.H, self.Dk, self.Dv), torch.float32)}

    def forward(self, q, f_raw, v, cache):
        T, H, Dk = q.shape[0], self.H, self.Dk
        r, v = F.silu(q.float()), v.float()
        low = self.lower.view(H, Dk)
        f = low + (1.0 - low) * torch.sigmoid(f_raw.float() + self.f_bias.view(H, Dk))
        out = torch.zeros(T, H, self.Dv, dtype=torch.float32, device=q.device)
        S_all = cache["state"]
        for b, slot, r0, nq, start in _spans(_ctx()):
            S = S_all[slot].clone() if start > 0 else torch.zeros_like(S_all[slot])
            for t in range(r0, r0 + nq):
                S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S, r[t])
            S_all[slot] = S
        return (_unit_rms(out, self.eps) * self.norm_weight).reshape(T, H * self.Dv).to(q.dtype)


class ShortConv(nn.Module):
    def __init__(self, channels, taps, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))

    def forward(self, x, conv_state):
        keep = self.taps - 1
        y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        for b, slot, r0, nq, start in _spans(_ctx()):
            past = conv_state[slot].float() if start > 0 else torch.zeros(keep, x.shape[1], device=x.device)
            if 0 < start < keep:
                past = past.clone()
                past[:keep - start] = 0
            seq = torch.cat([past, x[r0:r0 + nq].float()], dim=0)
            acc = torch.zeros(nq, x.shape[1], device=x.device)
            for j in range(self.taps):
                acc += seq[j:j + nq] * self.weight[:, j]
            y[r0:r0 + nq] = acc.to(x.dtype)
            if keep:
                conv_state[slot] = seq[seq.shape[0] - keep:].to(conv_state.dtype)
        return y


def _scaled_freqs(dims, base, scaling):
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave > orig / low:
                f = f / factor
            elif wave >= orig / high:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float32)


class KeyTiedAttention(nn.Module):
    def __init__(self, num_heads, num_kv_heads, head_dim, scale, eps, rot_dims=0, rot_base=10000.0, rot_scaling=None,
                 device=None):
        super().__init__()
        self.H, self.G, self.D = num_heads, num_kv_heads, head_dim
        self.scale, self.eps, self.rot_dims = float(scale), float(eps), int(rot_dims)
        f32 = dict(dtype=torch.float32, device=device)
        self.q_norm = nn.Parameter(torch.ones(head_dim, **f32))
        self.k_norm = nn.Parameter(torch.ones(head_dim, **f32))
        self.register_buffer("freq", _scaled_freqs(rot_dims, rot_base, rot_scaling).to(device) if rot_dims else None,
                             persistent=False)

    def forward(self, q, k, positions, k_cache, v_cache):
        ctx = _ctx()
        dt, T, H, G, D = q.dtype, q.shape[0], self.H, self.G, self.D
        qn, kn = _unit_rms(q.float(), self.eps) * self.q_norm, _unit_rms(k.float(), self.eps) * self.k_norm
        if self.rot_dims:
            qn, kn = _turn(qn, positions, self.freq, self.rot_dims), _turn(kn, positions, self.freq, self.rot_dims)
        qn, kn = qn.to(dt), kn.to(dt)
        bs = k_cache.shape[1]
        slots = ctx.slot_mapping.long()
        k_cache.view(-1, G, D)[slots] = kn
        v_cache.view(-1, G, D)[slots] = k
        cu_q, cu_k = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist()
        out = torch.zeros(T, H, D, dtype=torch.float32, device=q.device)
        for b in range(len(cu_q) - 1):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            pos_k = torch.arange(nk, device=q.device)
            rows = ctx.block_tables[b].long()[pos_k // bs] * bs + pos_k % bs
            kk, vv = k_cache.view(-1, G, D)[rows].float(), v_cache.view(-1, G, D)[rows].float()
            pos_q = nk - nq + torch.arange(nq, device=q.device)
            vis = pos_k[None, :] <= pos_q[:, None]
            qq = qn[cu_q[b]:cu_q[b + 1]].float()
            for h in range(H):
                g = h // (H // G)
                s = (qq[:, h] @ kk[:, g].t() * self.scale).masked_fill(~vis, float("-inf"))
                out[cu_q[b]:cu_q[b + 1], h] = torch.softmax(s, dim=-1) @ vv[:, g]
        return out.reshape(T, H * D).to(dt)


class GroupedSigmoidRouter(nn.Module):
    def __init__(self, experts, top, groups=1, keep_groups=1, device=None):
        super().__init__()
        self.E, self.top, self.groups, self.keep = int(experts), int(top), int(groups), int(keep_groups)
        self.correction = nn.Parameter(torch.zeros(experts, dtype=torch.float32, device=device))

    def forward(self, logits):
        s = torch.sigmoid(logits.float())
        choice = s + self.correction if self.correction is not None else s.clone()
        if self.groups > 1:
            per = choice.view(-1, self.groups, self.E // self.groups)
            merit = per.topk(min(2, per.shape[-1]), dim=-1).values.sum(-1)
            best = merit.topk(self.keep, dim=-1).indices
            allowed = torch.zeros_like(merit, dtype=torch.bool).scatter_(1, best, True)
            choice = per.masked_fill(~allowed[:, :, None], float("-inf")).reshape(-1, self.E)
        ids = choice.topk(self.top, dim=-1).indices
        return ids.to(torch.int32), s.gather(1, ids)


class SquaredReluExperts(nn.Module):
    def forward(self, h, ids, weights, up, down):
        T, top, dt = h.shape[0], ids.shape[1], h.dtype
        idx = ids.long()
        out = torch.zeros(T, top, down.shape[1], dtype=torch.float32, device=h.device)
        for e in idx.unique().tolist():
            t, j = (idx == e).nonzero(as_tuple=True)
            y = (torch.relu(F.linear(h[t], up[e]).float()) ** 2).to(dt)
            out[t, j] = F.linear(y, down[e]).float() * weights[t, j][:, None]
        return out
