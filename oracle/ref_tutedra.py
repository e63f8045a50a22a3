"""Oracle (test infrastructure): a plain, slow restatement of the Tutedra design, one function per mechanism,
whole sequences at a time, no cache and no batching.  It shares nothing with the product path: tests compare
the engine (paged cache, state slots, chunked prompts, mixed batches, HIP kernels) with these functions.

`dtype=torch.float32` computes everything in 32-bit.  With `torch.bfloat16` the matrix products and the short
convolutions take bfloat16 operands (fp32 accumulation, bfloat16 result) and everything the design keeps in 32-bit
stays there: the residual stream, norms, rotary angles, attention scores and weights, router scores, and both
recurrences with their gates, decays and running maxima.

A model is (cfg, weights): cfg the parsed config.json, weights a dict name -> tensor as stored.

The design in short.  x_0 = embed[token] + bigram[hash(previous token, token)], not normed.  Every layer is pre-norm with
one-plus norm weights and a per-column scale on each sublayer's output:
    h = norm1(x);  h <- h + (h_prev - h) * shift;  x += ls1 * mixer(h);  x += ls2 * ff(norm2(x)).
The mixer is a stabilised matrix memory with exponential gates (`mlstm`), a keyless gated linear recurrence that writes one
minus its forget gate (`hgrn2`), or softmax attention that reads its values from its un-normed keys, with a short convolution
behind the q / k projections, per-head q / k norms and scaled rotary frequencies (`attention`).  The feed-forward is
dense with a polynomial-of-norms activation, or a mixture of squared-ReLU experts with sigmoid scores, a selection
bias, group-limited choice and a gated shared expert.  logits = embed rmsnorm(x).
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


def one_plus_norm(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w.float())


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------------------------ embedding
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    return [buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets for t, tok in enumerate(tokens)]


def embed(cfg, w, tokens):
    x = w["embed"][torch.tensor(tokens)].float()
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        rows = bigram_rows(tokens, int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))
        x = x + w["bigram"][torch.tensor(rows)].float()
    return x


# ------------------------------------------------------------------------------------------ token shift
def token_shift(h, mu):
    """h_t + (h_(t-1) - h_t) * mu per column, the row before the first being zero; reads the un-shifted rows."""
    h = h.float()
    prev = torch.cat([torch.zeros(1, h.shape[1]), h[:-1]], dim=0)
    return h + (prev - h) * mu.float()


# ------------------------------------------------------------------------------------------ convolution, rotary
def causal_conv(u, w, dtype=torch.float32):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start; result in dtype."""
    T, C = u.shape
    taps = w.shape[1]
    u, w = u.to(dtype).float(), w.to(dtype).float()
    y = torch.zeros(T, C)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y.to(dtype)


def rotary_frequencies(rot):
    """f_i = base^(-2i/dims), then the three-band rescaling by wavelength: short waves keep f, long waves take
    f / factor, the band between blends the two linearly in original / wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wave = 2.0 * math.pi / f
            if wave < orig / high:
                pass
            elif wave > orig / low:
                f = f / factor
            else:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float32)


def rotate_halves(x, positions, freq):
    """x [T, heads, D]: the first 2 len(freq) dimensions turn, pair (i, i + len(freq)) by position * freq[i]."""
    half = freq.numel()
    if half == 0:
        return x.float()
    ang = positions.to(torch.float32)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x = x.float()
    out = x.clone()
    a, b = x[..., :half], x[..., half:2 * half]
    out[..., :half] = a * c - b * s
    out[..., half:2 * half] = b * c + a * s
    return out


# ------------------------------------------------------------------------------------------ mixers
def mlstm(m, w, p, h, eps, dtype):
    """Matrix memory with exponential gating.  Per head, with log gates i_t (input) and f_t (forget) and a running
    maximum m_t that keeps the exponentials bounded (m_0 = 0):
        m_t = max(f_t + m_(t-1), i_t)
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t the same with k_t alone
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
    Both gate pre-activations are soft-capped; the forget gate is a log-sigmoid of its capped value."""
    T = h.shape[0]
    H, D, Dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    q = linear(h, w[p + "q"], dtype).float().view(T, H, D) * D ** -0.5
    k = linear(h, w[p + "k"], dtype).float().view(T, H, D)
    v = linear(h, w[p + "v"], dtype).float().view(T, H, Dv)
    gi = cap * torch.tanh((linear(h, w[p + "i"], dtype).float() + w[p + "i.b"].float()) / cap)
    gf = F.logsigmoid(cap * torch.tanh((linear(h, w[p + "f"], dtype).float() + w[p + "f.b"].float()) / cap))
    S, n, mx = torch.zeros(H, D, Dv), torch.zeros(H, D), torch.zeros(H)
    o = torch.zeros(T, H, Dv)
    for t in range(T):
        m_new = torch.maximum(gf[t] + mx, gi[t])
        keep, write = torch.exp(gf[t] + mx - m_new), torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + write[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + write[:, None] * k[t]
        mx = m_new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den[:, None]
    o = rms_unit(o, eps).reshape(T, H * Dv) * w[p + "norm"].float()
    o = o * torch.sigmoid(linear(h, w[p + "g"], dtype).float())
    return linear(o.to(dtype), w[p + "o"], dtype)


def hgrn2(m, w, p, h, eps, dtype):
    """Gated linear recurrence with the forget gate tied to the write: per head and key channel a gate f in
    [lower, 1), S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t with q = silu(W_q h)."""
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = F.silu(linear(h, w[p + "q"], dtype).float()).to(dtype).float().view(T, H, D)
    v = linear(h, w[p + "v"], dtype).float().view(T, H, Dv)
    low = w[p + "lower"].float()
    f = (low + (1.0 - low) * torch.sigmoid(linear(h, w[p + "f"], dtype).float() + w[p + "f.b"].float())).view(T, H, D)
    S = torch.zeros(H, D, Dv)
    o = torch.zeros(T, H, Dv)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms_unit(o, eps) * w[p + "norm"].float()
    return linear(o.reshape(T, H * Dv).to(dtype), w[p + "o"], dtype)


def attention(m, w, p, h, eps, dtype):
    """Causal softmax attention, grouped query heads; the value of a token is its key as the convolution leaves it
    (ahead of the per-head norm and the rotary)."""
    T = h.shape[0]
    H, G, D = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    pos = torch.arange(T)
    q, k = linear(h, w[p + "q"], dtype), linear(h, w[p + "k"], dtype)
    if p + "q.conv" in w:
        q, k = causal_conv(q, w[p + "q.conv"], dtype), causal_conv(k, w[p + "k.conv"], dtype)
    v = k.float().view(T, G, D)
    q = rms_unit(q.float().view(T, H, D), eps) * w[p + "q.norm"].float()
    k = rms_unit(k.float().view(T, G, D), eps) * w[p + "k.norm"].float()
    rot = m.get("rot")
    if rot:
        freq = rotary_frequencies(rot)
        q, k = rotate_halves(q, pos, freq), rotate_halves(k, pos, freq)
    q, k = q.to(dtype).float(), k.to(dtype).float()
    visible = pos[None, :] <= pos[:, None]
    out = torch.zeros(T, H, D)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].t()) * float(m["scale"])
        a = torch.softmax(s.masked_fill(~visible, float("-inf")), dim=-1)
        out[:, hh] = a @ v[:, g]
    return linear(out.reshape(T, H * D).to(dtype), w[p + "o"], dtype)


# ------------------------------------------------------------------------------------------ feed-forward
def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with N(u) = u / rms(u) over the row."""
    a, b, c, e = (float(x) for x in coef.float())
    z = z.float()
    return a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e


def dense_ff(w, p, h, eps, dtype):
    return linear(poly_norm(linear(h, w[p + "up"], dtype), w[p + "act"], eps).to(dtype), w[p + "down"], dtype).float()


def squared_relu_expert(w, p, h, dtype):
    a = torch.relu(linear(h, w[p + "up"], dtype).float()) ** 2
    return linear(a.to(dtype), w[p + "down"], dtype).float()


def route(mlp, w, p, h32):
    """(chosen experts [T, top], their weights [T, top]).  Scores are sigmoids of the router logits; the CHOICE adds
    a per-expert correction and is restricted to the `keep` best consecutive blocks of experts (a block's merit: the
    sum of its top two biased scores); the weights are the plain scores of the chosen, as they are."""
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(F.linear(h32.float(), w[p + "router"].float()))
    choice = s + w[p + "correction"].float() if p + "correction" in w else s.clone()
    groups = r.get("groups")
    if groups and int(groups["count"]) > 1:
        n, keep = int(groups["count"]), int(groups["keep"])
        per = choice.view(-1, n, E // n)
        merit = per.topk(min(2, E // n), dim=-1).values.sum(-1)
        best = merit.topk(keep, dim=-1).indices
        allowed = torch.zeros_like(merit, dtype=torch.bool).scatter_(1, best, True)
        choice = per.masked_fill(~allowed[:, :, None], float("-inf")).reshape(-1, E)
    ids = choice.topk(top, dim=-1).indices
    return ids, s.gather(1, ids)


def moe_ff(mlp, w, p, h32, dtype):
    h = h32.to(dtype)
    ids, weights = route(mlp, w, p, h)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0])
    for t in range(h.shape[0]):
        for e, g in zip(ids[t].tolist(), weights[t].tolist()):
            out[t] += g * squared_relu_expert(w, f"{p}e{e}.", h[t:t + 1], dtype)[0]
    if p + "shared.up" in w:
        gate = torch.sigmoid(linear(h, w[p + "shared.sg"], dtype).float())
        out = out + gate * squared_relu_expert(w, p + "shared.", h, dtype)
    return out


# ------------------------------------------------------------------------------------------ the model
MIXERS = {"mlstm": mlstm, "hgrn2": hgrn2, "attention": attention}


def forward(cfg, weights, tokens, dtype=torch.float32):
    """Returns (logits [T, vocab] float32, the residual stream after every layer [layers, T, width])."""
    eps = float(cfg["norm"]["eps"])
    w = weights
    x = embed(cfg, w, tokens)
    streams = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = one_plus_norm(x, w[p + "norm1"], eps)
        if p + "shift" in w:
            h = token_shift(h.to(dtype), w[p + "shift"])
        y = MIXERS[L["type"]](L["mixer"], w, p + "mix.", h.to(dtype), eps, dtype).float()
        x = x + (y * w[p + "ls1"].float() if p + "ls1" in w else y)
        mlp = L.get("mlp")
        if mlp is not None:
            h = one_plus_norm(x, w[p + "norm2"], eps)
            y = dense_ff(w, p + "mlp.", h.to(dtype), eps, dtype) if mlp["kind"] == "dense" else moe_ff(mlp, w, p + "mlp.", h, dtype)
            x = x + (y * w[p + "ls2"].float() if p + "ls2" in w else y)
        streams.append(x.clone())
    logits = linear(one_plus_norm(x, w["final.norm"], eps).to(dtype), w["embed"], dtype).float()
    return logits, torch.stack(streams)
