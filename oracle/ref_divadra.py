"""Oracle (test infrastructure): a plain, slow restatement of the Divadra design, one function per mechanism,
whole sequences at a time, no cache and no batching.  It shares nothing with the product path: tests compare
the engine (paged cache, state slots, chunked prompts, mixed batches, HIP kernels) with these functions.

`dtype=torch.float32` computes everything in 32-bit.  With `torch.bfloat16` the matrix products take bfloat16
operands (fp32 accumulation, bfloat16 result) and everything the design keeps in 32-bit stays there: the residual
stream, norms, rotary angles, attention scores and weights, and both recurrences with their decays and gates.

A model is (cfg, weights): cfg the parsed config.json, weights a dict name -> tensor as stored.

The design in short.  x_0 = rmsnorm(embed[token] + bigram[hash(previous token, token)]).  Every layer has two norms of
the same stream, a = norm1(x) and b = norm2(x); each sublayer reads its input plus a short causal convolution of it;
x += mixer(a + conv1(a)) + ff(b + conv2(b)).  The mixer is either a Mamba-2 state-space layer or two mixers side by
side (sigmoid attention inside fixed chunks with rotated values, and an RWKV-style decayed outer-product memory),
whose outputs are each RMS-normed and averaged.  The feed-forward is dense (squared ReLU) or a set of small gated
experts that a table assigns to every token id.  logits = head rmsnorm(x).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def linear(x, w, dtype=torch.float32):
    return F.linear(x.to(dtype), w.to(dtype))


def rms_unit(x, eps):
    x = x.float()
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w.float()


def causal_conv(h, w, bias=None):
    """h [T, C], w [C, taps]: out_t = sum_j w[:, j] h_(t - taps + 1 + j) (+ bias), zeros before the start."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros(T, C) if bias is None else bias.float().expand(T, C).clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j].float() * h[s].float()
    return out


# ------------------------------------------------------------------------------------------ embedding
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table per position: a hash of (previous token, token); the first token takes the extra
    last row."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def embed(cfg, weights, tokens):
    x = weights["embed"][torch.tensor(tokens)].float()
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        rows = bigram_rows(tokens, int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))
        x = x + weights["bigram"][torch.tensor(rows)].float()
    return rms_norm(x, weights["embed.norm"], cfg["norm"]["eps"])


# ------------------------------------------------------------------------------------------ rotary
def rotate_halves(x, positions, dims, base, sign=1.0):
    """x [T, ..., D]: the first `dims` dimensions turn, pair (i, i + dims/2) by sign * position * base^(-2i/dims)."""
    if dims == 0:
        return x.float()
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float32)
    ang = positions.to(torch.float32)[:, None] * f[None, :] * sign
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    x = x.float()
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------ mixers
def chunk_sigmoid_attention(m, w, p, h, eps, dtype):
    """Grouped-query attention inside fixed chunks of positions: a key j is visible to query i when j <= i and both
    lie in the same chunk (counted from position 0).  The weight of a visible key is sigmoid(score + bias of the
    head), not normalised over keys.  Values are rotated by their own position before they are summed, and the sum
    is rotated back by the query's position."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    rot = m.get("rot") or {}
    rot_dims, base, size = int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), int((m.get("mask") or {}).get("size", 0))
    pos = torch.arange(T)
    q = rms_norm(linear(h, w[p + "q"], dtype), w[p + "q.norm"], eps).view(T, H, D)
    k = rms_norm(linear(h, w[p + "k"], dtype), w[p + "k.norm"], eps).view(T, G, D)
    v = linear(h, w[p + "v"], dtype).view(T, G, Dv)
    q = rotate_halves(q, pos, rot_dims, base).to(dtype).float()
    k = rotate_halves(k, pos, rot_dims, base).to(dtype).float()
    v = rotate_halves(v, pos, Dv, base).to(dtype).float()
    visible = pos[None, :] <= pos[:, None]
    if size:                                  # (no mask in the configuration: plain causal)
        visible = visible & ((pos[None, :] // size) == (pos[:, None] // size))
    out = torch.zeros(T, H, Dv)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].t()) * float(m["scale"]) + w[p + "pb"][hh].float()
        a = torch.sigmoid(s) * visible
        out[:, hh] = a @ v[:, g]
    out = rotate_halves(out, pos, Dv, base, sign=-1.0)
    return linear(out.reshape(T, H * Dv).to(dtype), w[p + "o"], dtype)


def decayed_memory(m, w, p, h, eps, dtype):
    """RWKV-style time mixing: every projection reads its own blend of the current and the previous input; per head a
    memory S [D, D] of decayed outer products k v^T is read with r, the current token's own product entering with a
    bonus u instead of through the memory."""
    T = h.shape[0]
    H, D = int(m["heads"]), int(m["dim"])
    h = h.float()
    prev = torch.cat([torch.zeros(1, h.shape[1]), h[:-1]], dim=0)
    mix = lambda s: (h + (prev - h) * w[p + "mu." + s].float()).to(dtype)
    r = linear(mix("r"), w[p + "r"], dtype).float().view(T, H, D)
    k = linear(mix("k"), w[p + "k"], dtype).float().view(T, H, D)
    v = linear(mix("v"), w[p + "v"], dtype).float().view(T, H, D)
    gate = F.silu(linear(mix("g"), w[p + "g"], dtype).float())
    low = torch.tanh(linear(mix("w"), w[p + "w1"], dtype).float()).to(dtype)
    decay = torch.exp(-torch.exp(linear(low, w[p + "w2"], dtype).float() + w[p + "w0"].float())).view(T, H, D)
    u = w[p + "u"].float().view(H, D)
    S = torch.zeros(H, D, D)
    o = torch.zeros(T, H, D)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[t])
        S = decay[t][:, :, None] * S + kv
    o = rms_unit(o, eps).reshape(T, H * D) * w[p + "norm"].float() * gate
    return linear(o.to(dtype), w[p + "o"], dtype)


def parallel_mixer(m, w, p, h, eps, dtype):
    """Both mixers read the same input; each output is RMS-normed over the width; the result is their mean."""
    a = chunk_sigmoid_attention(m["left"], w, p + "left.", h, eps, dtype)
    b = decayed_memory(m["right"], w, p + "right.", h, eps, dtype)
    return 0.5 * (rms_norm(a, w[p + "left.out"], eps) + rms_norm(b, w[p + "right.out"], eps))


def mamba2(m, w, p, h, eps, dtype):
    """State-space duality layer: per head a state S [N, P] with a scalar decay exp(-exp(A_log) dt) per step,
    S <- decay S + dt B x^T, y = S^T C + D x; the gate silu(z) comes before the grouped RMS norm."""
    T = h.shape[0]
    Hh, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner, ng = Hh * P, int(m.get("norm_groups", 1))
    proj = linear(h, w[p + "in"], dtype)
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = F.silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"])).to(dtype).float()
    x = xbc[:, :inner].view(T, Hh, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = F.softplus(dt.float() + w[p + "dt_bias"].float())
    rate = torch.exp(w[p + "A_log"].float())
    per = Hh // G
    S = torch.zeros(Hh, N, P)
    y = torch.zeros(T, Hh, P)
    for t in range(T):
        Bh, Ch = B[t].repeat_interleave(per, dim=0), C[t].repeat_interleave(per, dim=0)
        S = torch.exp(-rate * dt[t])[:, None, None] * S + dt[t][:, None, None] * Bh[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, Ch) + w[p + "D"].float()[:, None] * x[t]
    y = y.reshape(T, inner) * F.silu(z.float())
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w[p + "norm"].float()
    return linear(y.to(dtype), w[p + "o"], dtype)


# ------------------------------------------------------------------------------------------ feed-forward
def dense_ff(w, p, h, dtype):
    a = torch.relu(linear(h, w[p + "up"], dtype).float()) ** 2
    return linear(a.to(dtype), w[p + "down"], dtype).float()


def table_experts(mlp, w, p, h, tokens, dtype):
    """Every token id owns `top` experts (a row of the table); each contributes with weight 1 / top."""
    top = int(mlp["router"]["top"])
    table = w[p + "table"]
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0])
    for t, tok in enumerate(tokens):
        for e in table[tok].tolist()[:top]:
            q = f"{p}e{e}."
            a = (F.silu(linear(h[t:t + 1], w[q + "gate"], dtype).float()) * linear(h[t:t + 1], w[q + "up"], dtype).float())
            out[t] += linear(a.to(dtype), w[q + "down"], dtype).float()[0] / top
    return out


# ------------------------------------------------------------------------------------------ the model
def forward(cfg, weights, tokens, dtype=torch.float32):
    """Returns (logits [T, vocab] float32, the residual stream after every layer [layers, T, width])."""
    eps = float(cfg["norm"]["eps"])
    w = weights
    x = embed(cfg, w, tokens)
    streams = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        a = rms_norm(x, w[p + "norm1"], eps)
        if p + "canon1" in w:
            a = a + causal_conv(a, w[p + "canon1"])
        a = a.to(dtype)
        if L["type"] == "mamba2":
            y = mamba2(L["mixer"], w, p + "mix.", a, eps, dtype).float()
        elif L["type"] == "parallel":
            y = parallel_mixer(L["mixer"], w, p + "mix.", a, eps, dtype)
        else:
            raise ValueError(L["type"])
        mlp = L.get("mlp")
        if mlp is not None:
            b = rms_norm(x, w[p + "norm2"], eps)
            if p + "canon2" in w:
                b = b + causal_conv(b, w[p + "canon2"])
            b = b.to(dtype)
            y = y + (dense_ff(w, p + "mlp.", b, dtype) if mlp["kind"] == "dense"
                     else table_experts(mlp, w, p + "mlp.", b, tokens, dtype))
        x = x + y
        streams.append(x.clone())
    logits = linear(rms_norm(x, w["final.norm"], eps).to(dtype), w["head"], dtype).float()
    return logits, torch.stack(streams)
