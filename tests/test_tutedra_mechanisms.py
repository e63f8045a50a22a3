"""Each Tutedra mechanism alone, against the plain functions of oracle/ref_tutedra.py, on inputs made so that a fault
shows: the model's own modules (built on the eager stand-in layers on the CPU and, marked gpu, on the HIP kernels in
float32) are driven step by step through a paged cache with stale pages and state slots that others used before, and
compared with the oracle's whole-sequence result.

  * embedding: no norm, the first token's extra row, the carried previous token across portions;
  * token shift: reads the row before it as it was BEFORE the blend, zeros in front of the first token, across portions;
  * attention: a peaked softmax (large score scale) so that one missing or misplaced key moves the output; one key far
    back that a query is aimed at; values that differ from the prepared keys; convolution taps that reach across
    portions and in front of the sequence's start; rescaled rotary frequencies in all three bands;
  * matrix memory: a first token written with a large input gate and kept by forget gates close to one, read hundreds of
    tokens later; gate pre-activations far beyond the cap; the denominator's floor exp(-m) with m below and above zero;
  * gated-write recurrence: lower bounds close to one keep a first token for hundreds of tokens;
  * routing: negative selection scores (a closed group must lose against them), groups of one expert, one group, top =
    all open experts; squared-ReLU experts with a gated shared expert; the polynomial activation; the scaled boundary."""
import math

import pytest
import torch

from nanovllm_amd.model import tutedra as M
from oracle import ref_tutedra as O
from test_divadra_mechanisms import close, rn, run_in_steps
from tutedra_util import layer_namespace

BACKENDS = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]
F32 = torch.float32


@pytest.fixture(params=BACKENDS)
def dev(request):
    return request.param


def load(module, w):
    """Checkpoint-named tensors `w` (no prefix) into a mixer module of the model."""
    params = dict(module.named_parameters())
    seen = set()

    def take(name):
        seen.add(name)
        return w[name]
    with torch.no_grad():
        module.place("", take)
        for ck, pn in module.names("", "").items():
            params[pn].copy_(take(ck))
    assert seen == set(w), set(w) - seen
    module.finalize()


def lin(g, o, i, gain=1.0):
    return rn(g, o, i, std=gain / math.sqrt(i))


# ------------------------------------------------------------------------------------------------ embedding, shift
def test_embedding_is_not_normed_and_carries_the_previous_token(dev):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(1)
    V, W, buckets = 50, 24, 13
    cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": 7, "mul_cur": 3}}}
    w = {"embed": rn(g, V, W, std=3.0), "bigram": rn(g, buckets + 1, W, std=2.0)}
    emb = L.HashedBigramEmbedding(V, W, buckets, 7, 3, 1e-5, dtype=F32, device=dev, normed=False)
    assert emb.norm is None
    with torch.no_grad():
        emb.weight.copy_(w["embed"]), emb.bigram.copy_(w["bigram"])
    prev = torch.full((4,), 17, dtype=torch.int64, device=dev)            # what earlier owners left in the slots
    for seed, portions in ((2, [1]), (3, [5, 1, 2, 9]), (4, [30])):
        toks = torch.randint(0, V, (30,), generator=torch.Generator().manual_seed(seed))
        other = torch.randint(0, V, (6,), generator=torch.Generator().manual_seed(seed + 10))
        got = run_in_steps(lambda ids, pos: emb(ids, pos, prev), toks, portions, dev, other=other)
        close(got, O.embed(cfg, w, toks.tolist()), 1e-6)
    assert int(prev[1]) == int(toks[-1])
    plain = L.HashedBigramEmbedding(V, W, 0, 0, 0, 1e-5, dtype=F32, device=dev, normed=False)
    with torch.no_grad():
        plain.weight.copy_(w["embed"])
    close(run_in_steps(lambda ids, pos: plain(ids, pos, None), toks, [7, 1], dev), w["embed"][toks], 1e-6)


def test_token_shift_reads_the_unshifted_previous_row(dev):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(2)
    W, T = 20, 37
    mu = torch.rand(W, generator=g) * 1.5 - 0.25                           # also outside [0, 1]
    shift = L.TokenShiftMix(1, W, device=dev)
    with torch.no_grad():
        shift.mu[0].copy_(mu)
    h, other = rn(g, T, W), rn(g, 9, W)
    want = O.token_shift(h, mu)
    chained = h.clone()                                                   # the wrong reading: the row before AFTER its blend
    for t in range(1, T):
        chained[t] = h[t] + (chained[t - 1] - h[t]) * mu
    assert (want - chained).norm() > 0.1 * want.norm()
    for portions in ([T], [1], [2, 1, 9, 1, 1, 30]):
        state = torch.randn(4, W, device=dev)
        got = run_in_steps(lambda x, pos: shift(x, state)[0], h, portions, dev, other=other)
        close(got, want, 1e-6)


# ------------------------------------------------------------------------------------------------ attention
def attention_module(dev, g, W, heads, kv_heads, dim, conv, rot_dims, scaling, scale, base=40.0):
    L = layer_namespace(dev)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if conv:
        m["conv"] = conv
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = scaling
    w = {"q": lin(g, heads * dim, W), "k": lin(g, kv_heads * dim, W), "o": lin(g, W, heads * dim),
         "q.norm": rn(g, dim, std=0.3, mean=1.0), "k.norm": rn(g, dim, std=0.5, mean=1.5)}
    if conv:
        w["q.conv"], w["k.conv"] = rn(g, heads * dim, conv, std=0.6), rn(g, kv_heads * dim, conv, std=0.6)
    mc = M.TutedraConfig.from_dict({"vocab": 4, "width": W, "norm": {"eps": 1e-5}, "layers": [{"type": "attention", "mixer": m, "mlp": None}]})
    mod = M.TutedraAttention(mc.layers[0].mixer, W, 1e-5, L, F32, dev)
    load(mod, w)
    return mod, m, w


def attention_caches(mod, dev, nb, bs=4):
    m = mod.m
    kc, vc = torch.randn(nb, bs, m.kv_heads, m.dim, device=dev), torch.randn(nb, bs, m.kv_heads, m.dim, device=dev)   # stale pages
    caches = [(kc, vc)]
    if mod.conv is not None:
        caches.append({"conv": torch.randn(4, m.conv - 1, mod.channels, device=dev)})
    return caches


@pytest.mark.parametrize("heads,kv_heads,dim,conv,rot_dims,scaling", [
    (4, 2, 8, 3, 8, {"factor": 5.0, "low": 1.0, "high": 4.0, "original": 30}),      # all three bands at base 40
    (3, 1, 10, 5, 10, None), (2, 2, 6, 0, 0, None), (9, 1, 12, 1, 6, {"factor": 2.0, "low": 0.5, "high": 1.0, "original": 8}),
    (2, 1, 16, 2, 16, {"factor": 8.0, "low": 2.0, "high": 8.0, "original": 100})])
def test_attention_peaked_softmax_every_key_counts(dev, heads, kv_heads, dim, conv, rot_dims, scaling):
    """Score scale 5 / sqrt(dim): a few keys carry each row, so a key that is lost, shifted by one or rotated by a wrong
    frequency moves the output far beyond the bound.  Pages of 4, portions that cut taps and pages."""
    g = torch.Generator().manual_seed(3 + heads)
    W, T = 24, 150
    mod, m, w = attention_module(dev, g, W, heads, kv_heads, dim, conv, rot_dims, scaling, 5.0 / math.sqrt(dim))
    if scaling and heads == 4:
        f0 = O.rotary_frequencies({"dims": rot_dims, "base": 40.0})
        f1 = O.rotary_frequencies(m["rot"])
        assert f1[0] == f0[0] and abs(f1[-1] - f0[-1] / 5.0) < 1e-8 and f0[1] / 5.0 < f1[1] < f0[1]     # kept, blended, stretched
    h, other = rn(g, T, W), rn(g, 12, W)
    want = O.attention(m, w, "", h, 1e-5, F32)
    if conv > 1:
        unconv = O.attention({k: v for k, v in m.items() if k != "conv"}, {k: v for k, v in w.items() if "conv" not in k}, "", h, 1e-5, F32)
        assert (want - unconv).norm() > 0.3 * want.norm()
    for portions in ([T], [1], [2, 3, 1, 1, 64, 2, 70], [5, 3]):
        caches = attention_caches(mod, dev, 80)
        got = run_in_steps(lambda x, pos: mod(x, pos, caches), h, portions, dev, other=other)
        close(got, want)


@pytest.mark.parametrize("target,query,portions", [(0, 299, [1]), (3, 299, [296, 1]), (4, 298, [300]), (131, 260, [128, 4, 1]),
                                                    (299, 299, [7, 1])])
def test_attention_a_far_key_and_its_raw_value(dev, target, query, portions):
    """Identity-like projections (the input row IS [q | k]); query and target key are aligned and large in front of the
    norm weights, every other score is small: the output is the target's value, which is its key BEFORE norm and
    rotation (the norm weight is far from one, so the prepared key is another vector)."""
    g = torch.Generator().manual_seed(5)
    H, G, Dk, T = 2, 1, 8, 300
    W = (H + G) * Dk
    mod, m, w = attention_module(dev, g, W, H, G, Dk, 0, 0, None, 6.0 / Dk)
    eye = torch.eye(W)
    w["q"], w["k"] = eye[:H * Dk], eye[H * Dk:]
    w["q.norm"], w["k.norm"] = torch.ones(Dk), torch.full((Dk,), 2.0)
    w["o"][:, Dk:] = 0.0                                                  # only head 0 is looked at
    load(mod, w)
    aim = torch.tensor([1.0, -1.0, 1.0, 1.0, -1.0, 1.0, 1.0, -1.0])
    away = torch.tensor([1.0, 1.0, 1.0, -1.0, 1.0, 1.0, -1.0, -1.0])       # orthogonal to aim
    h = rn(g, T, W, std=0.3)
    h[:, H * Dk:] += 3.0 * away
    h[target, H * Dk:] = 3.0 * aim
    h[query, :Dk] = 3.0 * aim
    want = O.attention(m, w, "", h, 1e-5, F32)
    raw = O.linear(torch.cat([h[target, H * Dk:], torch.zeros(Dk)]), w["o"])
    assert (want[query] - raw).norm() < 0.02 * raw.norm()                 # head 0 reads the target's raw key, not the prepared one
    caches = attention_caches(mod, dev, 160)
    close(run_in_steps(lambda x, pos: mod(x, pos, caches), h, portions, dev, num_blocks=160, other=rn(g, 5, W)), want)


# ------------------------------------------------------------------------------------------------ recurrences
@pytest.mark.parametrize("heads,dim,vdim,cap", [(3, 10, 6, 12.0), (1, 33, 20, 2.0), (2, 64, 48, 30.0)])
def test_matrix_memory_reads_a_first_token_hundreds_of_tokens_later(dev, heads, dim, vdim, cap):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(7)
    W, T = 20, 260
    m = {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}
    w = {"q": lin(g, heads * dim, W, 1.5), "k": lin(g, heads * dim, W, 1.5), "v": lin(g, heads * vdim, W), "g": lin(g, heads * vdim, W),
         "i": lin(g, heads, W, 1.0), "f": lin(g, heads, W, 1.0), "i.b": rn(g, heads, std=0.5, mean=-1.0),
         "f.b": rn(g, heads, std=0.5, mean=7.0), "norm": rn(g, heads * vdim, std=0.1, mean=1.0), "o": lin(g, W, heads * vdim)}
    mod = M.TutedraMatrixMemory(M.MatrixMemoryConfig(heads, dim, vdim, cap), W, 1e-5, L, F32, dev)
    load(mod, w)
    h = rn(g, T, W, std=0.5)
    h[0] = 40.0 * w["i"][0] / w["i"][0].norm()                        # a large input gate (far beyond the cap) for head 0
    h[1] = -40.0 * w["i"][0] / w["i"][0].norm()                       # and one far below
    want = O.mlstm(m, w, "", h, 1e-5, F32)
    lost = O.mlstm(m, w, "", torch.cat([torch.zeros(1, W), h[1:]]), 1e-5, F32)
    if cap >= 8:           # (a cap of 2 bounds the forget gate by logsigmoid(2) a step: nothing lasts 260 of them)
        assert (want[-1] - lost[-1]).norm() > 0.05 * want[-1].norm()     # the last row does depend on the first token
    other = rn(g, 9, W)
    for portions in ([T], [1], [2, 255, 1], [129, 2, 64], [17]):
        cache = [{"state": torch.randn(4, heads, dim, vdim, device=dev), "normaliser": torch.randn(4, heads, dim, device=dev),
                  "maximum": torch.randn(4, heads, device=dev)}]
        got = run_in_steps(lambda x, pos: mod(x, pos, cache), h, portions, dev, num_blocks=140, other=other)
        close(got, want)


def test_matrix_memory_running_maximum_starts_at_zero_and_floors_the_denominator(dev):
    """Input gates far below zero at the start: the maximum stays 0 (its initial value is 0, not -inf), the
    normaliser is tiny and exp(-m) = 1 is the denominator; later large gates lift m and the floor falls away."""
    L, g = layer_namespace(dev), torch.Generator().manual_seed(8)
    W, T, heads, dim, vdim = 12, 40, 2, 6, 5
    m = {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": 12.0}
    w = {"q": lin(g, heads * dim, W), "k": lin(g, heads * dim, W), "v": lin(g, heads * vdim, W), "g": lin(g, heads * vdim, W),
         "i": torch.zeros(heads, W), "f": torch.zeros(heads, W), "i.b": torch.tensor([-8.0, -8.0]), "f.b": torch.tensor([2.0, -2.0]),
         "norm": torch.ones(heads * vdim), "o": lin(g, W, heads * vdim)}
    w["i"][:, 0] = 1.0
    mod = M.TutedraMatrixMemory(M.MatrixMemoryConfig(heads, dim, vdim, 12.0), W, 1e-5, L, F32, dev)
    load(mod, w)
    h = rn(g, T, W, std=0.5)
    h[:, 0] = 0.0
    h[20:, 0] = 14.0                                                    # i = 12 tanh(6 / 12) = +5.5 from row 20 on
    want = O.mlstm(m, w, "", h, 1e-5, F32)
    assert torch.isfinite(want).all()
    for portions in ([T], [1], [19, 2, 1]):
        cache = [{"state": torch.randn(4, heads, dim, vdim, device=dev), "normaliser": torch.randn(4, heads, dim, device=dev),
                  "maximum": torch.full((4, heads), 9.0, device=dev)}]
        got = run_in_steps(lambda x, pos: mod(x, pos, cache), h, portions, dev, other=rn(g, 4, W))
        close(got, want)
    assert float(cache[0]["maximum"][1].detach().min()) > 3.0                     # the carried maximum of the main sequence


@pytest.mark.parametrize("heads,dim,vdim", [(2, 12, 9), (1, 40, 64), (3, 64, 17)])
def test_gated_write_recurrence_keeps_a_first_token(dev, heads, dim, vdim):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(9)
    W, T = 20, 240
    m = {"heads": heads, "dim": dim, "vdim": vdim}
    w = {"q": lin(g, heads * dim, W, 1.5), "f": lin(g, heads * dim, W, 1.5), "v": lin(g, heads * vdim, W),
         "f.b": rn(g, heads * dim, std=1.0, mean=2.0), "lower": 0.97 + 0.03 * torch.rand(heads * dim, generator=g),
         "norm": rn(g, vdim, std=0.2, mean=1.0), "o": lin(g, W, heads * vdim)}
    w["lower"][::3] = 0.0                                                 # and channels without a bound
    mod = M.TutedraGatedWrite(M.GatedWriteConfig(heads, dim, vdim), W, 1e-5, L, F32, dev)
    load(mod, w)
    h = rn(g, T, W, std=0.5)
    h[0] = 30.0 * w["v"][0] / w["v"][0].norm()
    want = O.hgrn2(m, w, "", h, 1e-5, F32)
    lost = O.hgrn2(m, w, "", torch.cat([torch.zeros(1, W), h[1:]]), 1e-5, F32)
    assert (want[-1] - lost[-1]).norm() > 0.05 * want[-1].norm()
    other = rn(g, 9, W)
    for portions in ([T], [1], [2, 235, 1], [129, 2, 64]):
        cache = [{"state": torch.randn(4, heads, dim, vdim, device=dev)}]
        got = run_in_steps(lambda x, pos: mod(x, pos, cache), h, portions, dev, num_blocks=140, other=other)
        close(got, want)


# ------------------------------------------------------------------------------------------------ feed-forward, boundary
@pytest.mark.parametrize("experts,top,groups,keep,shared,correction", [
    (10, 3, 2, 1, 10, -2.0), (6, 2, 6, 3, 0, 0.0), (5, 5, 1, 1, 7, -1.0), (12, 4, 4, 2, 3, None), (7, 1, 0, 0, 0, 0.5), (70, 6, 7, 3, 5, -0.7)])
def test_routed_experts_with_groups_and_a_gated_shared_expert(dev, experts, top, groups, keep, shared, correction):
    """Corrections around `correction` (negative: every selection score of an open group can lie below zero, so a closed
    group must be shut out altogether rather than scored 0)."""
    L, g = layer_namespace(dev), torch.Generator().manual_seed(13 + experts)
    W, ff, T = 20, 12, 45
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if groups:
        mlp["router"]["groups"] = {"count": groups, "keep": keep}
    w = {"router": rn(g, experts, W, std=0.8)}
    if correction is not None:
        w["correction"] = rn(g, experts, std=0.2, mean=correction)
    for e in range(experts):
        w[f"e{e}.up"], w[f"e{e}.down"] = rn(g, ff, W, std=0.4), rn(g, W, ff, std=0.3)
    if shared:
        mlp["shared"] = {"ff": shared}
        w["shared.up"], w["shared.down"], w["shared.sg"] = rn(g, shared, W, std=0.4), rn(g, W, shared, std=0.3), rn(g, 1, W, std=0.5)
    c = M.TutedraConfig.from_dict({"vocab": 4, "width": W, "norm": {"eps": 1e-5},
                                   "layers": [{"type": "hgrn2", "mixer": {"heads": 1, "dim": 4, "vdim": 4}, "mlp": mlp}]}).layers[0].mlp
    mod = M.TutedraMoE(c, W, L, F32, dev)
    with torch.no_grad():
        mod.router_weight.copy_(w["router"])
        if correction is not None:
            mod.router.correction.copy_(w["correction"])
        else:
            mod.router.correction = None
        for e in range(experts):
            mod.up[e].copy_(w[f"e{e}.up"]), mod.down[e].copy_(w[f"e{e}.down"])
        if shared:
            mod.shared_in.weight[:shared].copy_(w["shared.up"]), mod.shared_in.weight[shared].copy_(w["shared.sg"][0])
            mod.shared_down.weight.copy_(w["shared.down"])
    h = rn(g, T, W)
    ids, wts = O.route(mlp, w, "", h)
    got_ids, got_w = mod.router((h @ w["router"].t()).to(dev))
    assert got_ids.cpu().sort(1).values.tolist() == ids.sort(1).values.tolist()
    close(got_w.cpu().sort(1).values, wts.sort(1).values, 1e-6)
    if groups > 1 and correction is not None and correction <= -1.0:
        scores = torch.sigmoid(h @ w["router"].t()) + w["correction"]
        assert (scores.gather(1, ids) < 0).any()
    out = mod(h.to(dev), h.to(dev))
    x = torch.zeros(T, W, device=dev)
    L.stream_boundary_scaled(x, **out)
    close(x.cpu(), O.moe_ff(mlp, w, "", h, F32))


def test_dense_ff_polynomial_activation_and_scaled_boundary(dev):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(15)
    W, ff, T = 28, 50, 11
    w = {"up": rn(g, ff, W, std=0.3), "down": rn(g, W, ff, std=0.3), "act": torch.tensor([0.7, -0.4, 0.25, 0.1])}
    c = M.FeedForwardConfig("dense", ff)
    mod = M.TutedraDenseFF(c, W, 1e-5, L, F32, dev)
    with torch.no_grad():
        mod.up.weight.copy_(w["up"]), mod.down.weight.copy_(w["down"]), mod.act.coef.copy_(w["act"])
    h = rn(g, T, W)
    close(mod(h.to(dev), None)["add"].cpu(), O.dense_ff(w, "", h, 1e-5, F32))
    z = rn(g, 5, 300, std=3.0)
    close(mod.act(z.to(dev)).cpu(), O.poly_norm(z, w["act"], 1e-5), 1e-6)
    x, a1, a2, gate, parts = rn(g, T, W), rn(g, T, W), rn(g, T, W), rn(g, T, 3), rn(g, T, 3, W)
    ls, nw = rn(g, W, std=0.3, mean=0.7), rn(g, W, std=0.1)
    norm = L.OnePlusNorm(W, device=dev)
    with torch.no_grad():
        norm.weight.copy_(nw)
    norm.finalize()
    to = lambda t: t.to(dev)
    xd = to(x.clone())
    h32, hd = L.stream_boundary_scaled(xd, add=to(a1), gated=(to(a2), to(gate)[:, 1]), parts=to(parts), col_scale=to(ls),
                                       norm=norm.applied, eps=1e-5, out_dtype=F32, want_f32=True)
    want = x + ls * (a1 + torch.sigmoid(gate[:, 1:2]) * a2 + parts.sum(1))
    close(xd.cpu(), want, 1e-6)
    close(h32.cpu(), O.one_plus_norm(want, nw, 1e-5), 1e-6)
    close(hd.cpu(), O.one_plus_norm(want, nw, 1e-5), 1e-6)
    h32, hd = L.stream_boundary_scaled(xd, norm=norm.applied, eps=1e-5, out_dtype=F32)          # the first norm: nothing is added
    assert h32 is None
    close(xd.cpu(), want, 1e-6)
    close(hd.cpu(), O.one_plus_norm(want, nw, 1e-5), 1e-6)
    L.stream_boundary_scaled(xd, add=to(a1))                                                      # no scale, no norm
    close(xd.cpu(), want + a1, 1e-6)
