"""Each Divadra mechanism alone, against the plain functions of oracle/ref_divadra.py, on inputs made so that a fault
shows: the model's own modules (built on the eager stand-in layers on the CPU and, marked gpu, on the HIP kernels in
float32) are driven step by step through a paged cache with shuffled pages and state slots in any order, and compared
with the oracle's whole-sequence result.

  * bigram embedding: the first token's extra row, the carried previous token across portions, a slot that another
    sequence used before;
  * chunked sigmoid attention: one key made to stand out (a query aligned with it, every other weight pushed down by
    the head bias) just inside and just outside the query's chunk, at a page border, in a prompt and in decoding;
  * decayed memory and state-space scan: a first token scaled up and decays close to one, read hundreds of tokens
    later through the carried state; portions down to one token;
  * table experts: top = 1, top = experts, experts that get no token; squared ReLU; the two-norm boundary."""
import math

import pytest
import torch

import nanovllm_amd as nv
from divadra_util import layer_namespace, paged_context
from nanovllm_amd.model import divadra as D
from oracle import ref_divadra as O

BACKENDS = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]
F32 = torch.float32


@pytest.fixture(params=BACKENDS)
def dev(request):
    return request.param


def rn(g, *s, std=1.0, mean=0.0):
    return torch.randn(*s, generator=g) * std + mean


def fill(module, names, tensors):
    params = dict(module.named_parameters())
    with torch.no_grad():
        for ck, pn in names.items():
            p = params[pn]
            if p.shape != tensors[ck].shape:
                p.data = torch.empty(tensors[ck].shape, dtype=p.dtype, device=p.device)
            p.copy_(tensors[ck])
    module.finalize()


def run_in_steps(fn, rows, portions, dev, block_size=4, num_blocks=80, slot=1, other=None):
    """Feed `rows` [T, ...] of one sequence through fn(step rows, positions) in portions; beside it, optionally, rows
    of another sequence (`other`) in single tokens, to make every step a mixed batch.  Returns the outputs for `rows`."""
    outs, at, n_other = [], 0, 0
    sizes = list(portions)
    while at < rows.shape[0]:
        n = min(sizes.pop(0) if len(sizes) > 1 else sizes[0], rows.shape[0] - at)
        n_q, n_k, slots, x = [n], [at + n], [slot], [rows[at:at + n]]
        if other is not None and n_other < other.shape[0]:
            n_q, n_k, slots, x = [1] + n_q, [n_other + 1] + n_k, [slot + 1] + slots, [other[n_other:n_other + 1]] + x
            n_other += 1
        # the same seed every step: a sequence keeps its pages (tables are prefixes of one permutation per row order)
        ctx, pos = paged_context_stable(n_q, n_k, block_size, num_blocks, dev, slots)
        nv.set_context(ctx)
        y = fn(torch.cat(x).to(dev), pos)
        outs.append(y[-n:].float().cpu())
        at += n
    nv.set_context(None)
    return torch.cat(outs)


def paged_context_stable(n_qs, n_ks, block_size, num_blocks, dev, slots):
    """Like paged_context, but sequence b always owns the pages b, b + S, b + 2 S, ... reversed (S = 2): tables do not
    change between steps while rows and lengths do."""
    S = 2
    first = 0 if len(n_qs) == 2 else 1                 # the main sequence keeps its pages with or without a companion
    tables, slot_map, pos = [], [], []
    width = max(-(-n // block_size) for n in n_ks) + 1
    for i, (nq, nk) in enumerate(zip(n_qs, n_ks)):
        b = first + i
        row = [num_blocks - 1 - (b + S * j) for j in range(-(-nk // block_size))]
        tables.append(row + [-1] * (width - len(row)))
        for p in range(nk - nq, nk):
            slot_map.append(row[p // block_size] * block_size + p % block_size)
            pos.append(p)
    cu = lambda xs: torch.tensor([0] + torch.tensor(xs).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    ctx = nv.CacheContext(slot_mapping=torch.tensor(slot_map, dtype=torch.int32, device=dev), cu_seqlens_q=cu(n_qs),
                          cu_seqlens_k=cu(n_ks), max_seqlen_q=max(n_qs), max_seqlen_k=max(n_ks),
                          block_tables=torch.tensor(tables, dtype=torch.int32, device=dev), block_size=block_size,
                          state_slots=torch.tensor(slots, dtype=torch.int32, device=dev))
    return ctx, torch.tensor(pos, dtype=torch.int64, device=dev)


def close(got, want, tol=2e-5):
    err = ((got - want).norm() / want.norm().clamp_min(1e-30)).item()
    assert err < tol, err


# ------------------------------------------------------------------------------------------------ embedding
def test_bigram_embedding_first_row_carry_and_slot_reuse(dev):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(1)
    V, W, buckets = 50, 24, 13
    cfg = {"norm": {"eps": 1e-5}, "embedding": {"bigram": {"buckets": buckets, "mul_prev": 7, "mul_cur": 3}}}
    w = {"embed": rn(g, V, W), "bigram": rn(g, buckets + 1, W, std=2.0), "embed.norm": rn(g, W, std=0.1, mean=1.0)}
    emb = L.HashedBigramEmbedding(V, W, buckets, 7, 3, 1e-5, dtype=F32, device=dev)
    with torch.no_grad():
        emb.weight.copy_(w["embed"]), emb.bigram.copy_(w["bigram"]), emb.norm.copy_(w["embed.norm"])
    prev = torch.full((4,), 17, dtype=torch.int64, device=dev)            # what earlier owners left in the slots
    for seed, portions in ((2, [1]), (3, [5, 1, 2, 9]), (4, [30])):
        toks = torch.randint(0, V, (30,), generator=torch.Generator().manual_seed(seed))
        other = torch.randint(0, V, (6,), generator=torch.Generator().manual_seed(seed + 10))
        got = run_in_steps(lambda ids, pos: emb(ids, pos, prev), toks, portions, dev, other=other)
        close(got, O.embed(cfg, w, toks.tolist()), 1e-6)
    assert int(prev[1]) == int(toks[-1])
    first_rows = O.bigram_rows(toks.tolist(), buckets, 7, 3)
    assert first_rows[0] == buckets and max(first_rows[1:]) < buckets


# ------------------------------------------------------------------------------------------------ attention
def attention_setup(dev, chunk, H=2, G=1, Dk=8, Dv=6, rot=4, seed=5):
    """Identity-like projections: the input row IS [q | k | v], so a test can aim a query at a key."""
    L, g = layer_namespace(dev), torch.Generator().manual_seed(seed)
    W = H * Dk + G * Dk + G * Dv
    m = {"heads": H, "kv_heads": G, "dim": Dk, "vdim": Dv, "scale": 3.0 / Dk, "mask": {"size": chunk},
         "rot": {"dims": rot, "base": 50.0}}
    eye = torch.eye(W)
    w = {"q": eye[:H * Dk], "k": eye[H * Dk:H * Dk + G * Dk], "v": eye[H * Dk + G * Dk:], "o": rn(g, W, H * Dv, std=0.3),
         "q.norm": rn(g, H * Dk, std=0.1, mean=1.0), "k.norm": rn(g, G * Dk, std=0.1, mean=1.0), "pb": torch.tensor([-9.0] * H)}
    mc = D.DivadraConfig.from_dict({"vocab": 4, "width": W, "norm": {"eps": 1e-5},
                                    "layers": [{"type": "parallel", "mlp": None, "mixer": {"left": m, "right": {"heads": 1, "dim": 4}}}]})
    mod = D.DivadraChunkAttention(mc.layers[0].mixer[0], W, 1e-5, L, F32, dev)
    fill(mod, mod.names("", ""), w)
    return mod, m, w, W, g


@pytest.mark.parametrize("chunk,target,query", [(8, 16, 23), (8, 15, 23), (8, 16, 16), (12, 24, 27), (12, 23, 24), (0, 0, 39)])
def test_chunk_attention_one_key_stands_out_inside_and_outside(dev, chunk, target, query):
    """Every weight is sigmoid(small - 9) except query -> target, whose q and k rows are aligned and large before the
    norm's weights: inside the chunk the output is about the target's value, outside about nothing.  Pages of 4: the
    chunk edges 8, 16, 24 are page borders, 12 is not."""
    mod, m, w, W, g = attention_setup(dev, chunk)
    H, G, Dk, Dv = 2, 1, 8, 6
    T = 40
    h = rn(g, T, W, std=0.05)
    aim = torch.tensor([1.0, -1.0, 1.0, 1.0, -1.0, 1.0, 1.0, -1.0])
    h[:, H * Dk + G * Dk:] = rn(g, T, G * Dv)                        # values of ordinary size
    h[target, H * Dk:H * Dk + Dk] = aim
    h[query, :Dk] = aim
    h[query, Dk:2 * Dk] = aim
    want = O.chunk_sigmoid_attention(m, w, "", h, 1e-5, F32)
    inside = target <= query and (chunk == 0 or target // chunk == query // chunk)
    if target != query:
        plain = h.clone()
        plain[target, H * Dk:H * Dk + Dk] = 0.05 * aim.roll(1) * torch.tensor([1.0, 1, -1, 1, 1, -1, 1, 1])
        far = O.chunk_sigmoid_attention(m, w, "", plain, 1e-5, F32)[query]
        assert ((want[query] - far).norm() > 0.2 * want[query].norm()) == inside       # the target matters iff it is visible
    nb = 24
    for portions in ([T], [1], [query, 1, 3], [5, 3, 9]):
        kc = torch.randn(nb, 4, G, Dk, device=dev)                    # stale contents in every page
        vc = torch.randn(nb, 4, G, Dv, device=dev)
        got = run_in_steps(lambda x, pos: mod(x, pos, (kc, vc)), h, portions, dev, num_blocks=nb)
        close(got, want)


def test_chunk_attention_mixed_batch_and_long_chunks(dev):
    mod, m, w, W, g = attention_setup(dev, chunk=70, H=4, G=2, Dk=6, Dv=10, rot=6, seed=7)
    with torch.no_grad():
        mod.attn.head_bias.fill_(-2.0)
    w["pb"] = torch.full((4,), -2.0)
    h, other = rn(g, 150, W), rn(g, 20, W)
    want = O.chunk_sigmoid_attention(m, w, "", h, 1e-5, F32)
    for portions in ([67, 3, 1], [1], [150]):
        kc, vc = torch.zeros(80, 4, 2, 6, device=dev), torch.zeros(80, 4, 2, 10, device=dev)
        got = run_in_steps(lambda x, pos: mod(x, pos, (kc, vc)), h, portions, dev, other=other)
        close(got, want)


# ------------------------------------------------------------------------------------------------ recurrences
def test_decayed_memory_reads_a_first_token_hundreds_of_tokens_later(dev):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(9)
    W, H, Dh, rank, T = 20, 3, 12, 3, 260
    m = {"heads": H, "dim": Dh}
    n = H * Dh
    lin = lambda o, i, gain=1.0: rn(g, o, i, std=gain / math.sqrt(i))
    w = {s: lin(n, W, 1.5) for s in ("r", "k", "v", "g")}
    w.update({"mu." + s: torch.rand(W, generator=g) for s in ("r", "k", "v", "g", "w")})
    w.update({"w1": lin(rank, W), "w2": lin(n, rank), "w0": rn(g, n, std=0.3, mean=-7.0), "u": rn(g, H, Dh, std=0.5),
              "norm": rn(g, n, std=0.1, mean=1.0), "o": lin(W, n)})
    mod = D.DivadraTimeMix(D.TimeMixConfig(H, Dh), W, 1e-5, L, F32, dev)
    names = mod.names("", "")
    fill(mod, names, {k: v for k, v in w.items() if not k.startswith("mu.")})
    with torch.no_grad():
        for j, s in enumerate(mod._mixes):
            mod.shift.mu[j].copy_(w["mu." + s])
    h = rn(g, T, W, std=0.3)
    h[0] *= 30.0                                                       # decays of about exp(-exp(-7)): it stays in the memory
    want = O.decayed_memory(m, w, "", h, 1e-5, F32)
    lost = O.decayed_memory(m, w, "", torch.cat([torch.zeros(1, W), h[1:]]), 1e-5, F32)
    assert (want[-1] - lost[-1]).norm() > 0.3 * want[-1].norm()        # the last row does depend on the first token
    other = rn(g, 9, W)
    for portions in ([T], [1], [2, 255, 1], [129, 2, 64]):
        cache = {"prev": torch.randn(4, W, device=dev), "state": torch.randn(4, H, Dh, Dh, device=dev)}
        got = run_in_steps(lambda x, pos: mod(x, pos, cache), h, portions, dev, num_blocks=140, other=other)
        close(got, want)


@pytest.mark.parametrize("heads,vdim,state,groups,ng,conv", [(4, 6, 10, 2, 3, 4), (3, 16, 33, 1, 1, 2), (2, 20, 5, 2, 8, 1)])
def test_state_space_layer_reads_a_first_token_hundreds_of_tokens_later(dev, heads, vdim, state, groups, ng, conv):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(11)
    W, T = 24, 230
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": ng, "conv": conv}
    inner, ch = heads * vdim, heads * vdim + 2 * groups * state
    w = {"in": rn(g, 2 * inner + 2 * groups * state + heads, W, std=1.0 / math.sqrt(W)), "conv": rn(g, ch, conv, std=0.5),
         "conv.b": rn(g, ch, std=0.3), "dt_bias": rn(g, heads, std=0.5, mean=-3.0), "A_log": rn(g, heads, std=0.3, mean=-3.0),
         "D": rn(g, heads), "norm": rn(g, inner, std=0.1, mean=1.0), "o": rn(g, W, inner, std=1.0 / math.sqrt(inner))}
    mc = D.StateSpaceConfig(heads, vdim, state, groups, ng, conv)
    mod = D.DivadraStateSpace(mc, W, 1e-5, L, F32, dev)
    fill(mod, mod.names("", ""), w)
    h = rn(g, T, W, std=0.5)
    h[0] *= 8.0
    want = O.mamba2(m, w, "", h, 1e-5, F32)
    lost = O.mamba2(m, w, "", h[-100:], 1e-5, F32)                        # what a state lost 100 tokens ago would give
    assert (want[-1] - lost[-1]).norm() > 0.05 * want[-1].norm()
    other = rn(g, 7, W)
    for portions in ([T], [1], [2, 200, 1], [3, 2]):
        cache = [{"conv": torch.randn(4, conv - 1, ch, device=dev), "state": torch.randn(4, heads, state, vdim, device=dev)}]
        got = run_in_steps(lambda x, pos: mod(x, pos, cache)[0][0], h, portions, dev, num_blocks=140, other=other)
        close(got, want)


# ------------------------------------------------------------------------------------------------ feed-forward, boundary
@pytest.mark.parametrize("experts,top", [(5, 2), (4, 1), (3, 3), (40, 2)])
def test_table_experts(dev, experts, top):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(13)
    V, W, ff, T = 30, 20, 12, 45
    w = {"table": torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(V)]).to(torch.int32)}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rn(g, ff, W, std=0.4), rn(g, ff, W, std=0.4), rn(g, W, ff, std=0.3)
    mlp = {"router": {"experts": experts, "top": top}}
    mod = D.DivadraTableMoE(D.FeedForwardConfig("moe", ff, experts, top), V, W, L, F32, dev)
    with torch.no_grad():
        mod.table.copy_(w["table"])
        for e in range(experts):
            mod.gate_up[e].copy_(torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]))
            mod.down[e].copy_(w[f"e{e}.down"])
    toks = torch.randint(0, V, (T,), generator=g)
    h = rn(g, T, W)
    _, parts, scale = mod(h.to(dev), toks.to(dev))
    assert parts.shape == (T, top, W) and scale == 1.0 / top
    close(parts.sum(1).cpu() * scale, O.table_experts(mlp, w, "", h, toks.tolist(), F32))


def test_dense_ff_and_two_norm_boundary(dev):
    L, g = layer_namespace(dev), torch.Generator().manual_seed(15)
    W, ff, T = 28, 50, 11
    w = {"up": rn(g, ff, W, std=0.3), "down": rn(g, W, ff, std=0.3)}
    mod = D.DivadraDenseFF(D.FeedForwardConfig("dense", ff), W, L, F32, dev)
    with torch.no_grad():
        mod.up.weight.copy_(w["up"]), mod.down.weight.copy_(w["down"])
    h = rn(g, T, W)
    close(mod(h.to(dev), None)[0].cpu(), O.dense_ff(w, "", h, F32))
    x, a1, a2, parts, n1, n2 = rn(g, T, W), rn(g, T, W), rn(g, T, W), rn(g, T, 3, W), rn(g, T, W, std=5.0), rn(g, T, W, std=0.1)
    w1, w2, wa, wb = rn(g, W), rn(g, W), rn(g, W), rn(g, W)
    to = lambda t: t.to(dev)
    xd = to(x.clone())
    h32, hd = L.stream_boundary_pair(xd, adds=[to(a1), to(a2)], parts=to(parts), parts_scale=1 / 3, normed=[(to(n1), to(w1)), (to(n2), to(w2))],
                                     normed_mult=0.5, norms=[to(wa), to(wb)], eps=1e-5, out_dtype=F32)
    want = x + a1 + a2 + parts.sum(1) / 3 + 0.5 * (O.rms_norm(n1, w1, 1e-5) + O.rms_norm(n2, w2, 1e-5))
    close(xd.cpu(), want, 1e-6)
    close(h32.cpu(), torch.cat([O.rms_norm(want, wa, 1e-5), O.rms_norm(want, wb, 1e-5)], dim=1), 1e-6)
    close(hd.cpu(), O.rms_norm(want, wa, 1e-5), 1e-6)
    h32, hd = L.stream_boundary_pair(xd, norms=[to(wb)], eps=1e-5)
    assert hd is None
    close(h32.cpu(), O.rms_norm(want, wb, 1e-5), 1e-6)
