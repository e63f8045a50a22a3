"""GPU parity of the HIP layers Divadra is built from against their eager stand-ins (oracle/ref_divadra_modules.py),
layer by layer, in float32 and bfloat16, on a mixed step (prompt portions beside single rows, shuffled pages, state
slots in any order) with sizes that exercise the kernels' tails: widths that are no multiple of a vector, head sizes
between the register layouts, key size != value size, the MFMA tile kernel's head sizes with chunk edges inside its
tiles, experts that get no row."""
import numpy as np
import pytest
import torch

import nanovllm_amd as nv
from buvalix_util import paged_context
from oracle import ref_divadra_modules as R

pytestmark = pytest.mark.gpu
DEV = "cuda"


def hip_layers():
    from nanovllm_amd.model.divadra import _default_layers
    return _default_layers()


def rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-30)).item()


def tol(dt):
    return 3e-6 if dt == torch.float32 else 1e-2


@pytest.fixture(params=[torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def dt(request):
    return request.param


N_Q, N_K, SLOTS = [5, 1, 17, 2, 1], [5, 40, 30, 2, 9], [2, 0, 3, 1, 4]


@pytest.fixture
def step():
    ctx, pos = paged_context(N_Q, N_K, 8, 40, 1, DEV, slots=SLOTS)
    ctx.cu_seqlens_q_host = ctx.cu_seqlens_q.cpu().numpy()
    nv.set_context(ctx)
    yield sum(N_Q), pos
    nv.set_context(None)


def rn(g, *s, std=1.0, mean=0.0):
    return (torch.randn(*s, generator=g) * std + mean).to(DEV)


def pair(cls_name, *args, **kw):
    a, b = getattr(hip_layers(), cls_name)(*args, device=DEV, **kw), getattr(R, cls_name)(*args, device=DEV, **kw)
    g = torch.Generator().manual_seed(len(cls_name))
    with torch.no_grad():
        for (_, pa), (_, pb) in zip(a.named_parameters(), b.named_parameters()):
            v = rn(g, *pa.shape, std=0.3, mean=0.2).to(pa.dtype)
            pa.copy_(v), pb.copy_(v)
    return a, b


@pytest.mark.parametrize("W,buckets", [(96, 13), (100, 211), (2048, 7), (40, 0)])
def test_hashed_bigram_embedding(dt, step, W, buckets):
    T, _ = step
    V = 70
    a, b = pair("HashedBigramEmbedding", V, W, buckets, 31, 5, 1e-6, dtype=dt)
    g = torch.Generator().manual_seed(W)
    ids = torch.randint(0, V, (T,), generator=g).to(DEV)
    pos = step[1]
    sa = torch.randint(0, V, (6,), generator=g).to(DEV)
    sb = sa.clone()
    ya, yb = a(ids, pos, sa), b(ids, pos, sb)
    assert rel(ya, yb) < 3e-6 and (buckets == 0 or torch.equal(sa, sb))


@pytest.mark.parametrize("W", [96, 100, 2048, 520])
def test_stream_boundary_pair(dt, W):
    L, g, T = hip_layers(), torch.Generator().manual_seed(W), 9
    x, a1, a2, parts = rn(g, T, W), rn(g, T, W).to(dt), rn(g, T, 2 * W).to(dt)[:, W:], rn(g, T, 3, W)
    n1, n2, w1, w2, wa, wb = rn(g, T, W).to(dt), rn(g, T, W, std=9.0).to(dt), rn(g, W), rn(g, W), rn(g, W), rn(g, W)
    for kw in (dict(adds=[a1, a2], parts=parts, parts_scale=0.5, normed=[(n1, w1), (n2, w2)], normed_mult=0.5, norms=[wa, wb]),
               dict(adds=[a2], norms=[wa], out_dtype=dt, want_f32=False), dict(normed=[(n2, w2)], normed_mult=2.0),
               dict(parts=parts, norms=[wa, wb], out_dtype=dt)):
        xa, xb = x.clone(), x.clone()
        ra, rb = L.stream_boundary_pair(xa, eps=1e-6, **kw), R.stream_boundary_pair(xb, eps=1e-6, **kw)
        assert rel(xa, xb) < 2e-6
        for u, v, t in zip(ra, rb, (3e-6, tol(dt))):
            assert (u is None) == (v is None)
            assert u is None or (u.shape == v.shape and rel(u, v) < t)


@pytest.mark.parametrize("cols", [24, 1000])
def test_relu_squared(dt, cols):
    g = torch.Generator().manual_seed(cols)
    x = rn(g, 7, 2 * cols).to(dt)[:, cols:]
    assert rel(hip_layers().ReluSquared()(x), R.ReluSquared()(x)) < tol(dt)


@pytest.mark.parametrize("C,n", [(96, 5), (100, 1), (1030, 3)])
def test_token_shift_mix(dt, step, C, n):
    T, _ = step
    a, b = pair("TokenShiftMix", n, C)
    g = torch.Generator().manual_seed(C)
    h = rn(g, T, 2 * C).to(dt)[:, :C]
    sa = rn(g, 6, C).to(dt)
    sb = sa.clone()
    ya, yb = a(h, sa), b(h, sb)
    assert rel(ya, yb) < tol(dt) and torch.equal(sa, sb)


@pytest.mark.parametrize("H,Dk,Dv", [(3, 12, 12), (2, 64, 64), (2, 40, 24), (1, 130, 70), (5, 8, 33)])
def test_decay_memory(dt, step, H, Dk, Dv):
    T, _ = step
    a, b = pair("DecayMemory", H, Dk, Dv, 1e-6)
    g = torch.Generator().manual_seed(H * Dk)
    with torch.no_grad():
        a.w_bias.copy_(rn(g, H * Dk, mean=-2.0)), b.w_bias.copy_(a.w_bias)
    r, k, v = rn(g, T, H, Dk).to(dt), rn(g, T, H, Dk, std=0.5).to(dt), rn(g, T, H, Dv).to(dt)
    w_raw, gate = rn(g, T, H * Dk).to(dt), rn(g, T, H * Dv).to(dt)
    sa = rn(g, 6, H, Dk, Dv)
    sb = sa.clone()
    ya, yb = a(r, k, v, w_raw, gate, sa), b(r, k, v, w_raw, gate, sb)
    assert rel(ya, yb) < tol(dt) and rel(sa, sb) < 3e-6


@pytest.mark.parametrize("H,G,N,P", [(4, 2, 10, 6), (2, 1, 128, 64), (3, 3, 33, 20), (8, 1, 16, 100)])
def test_state_space_scan_and_group_norm(dt, step, H, G, N, P):
    T, _ = step
    a, b = pair("StateSpaceScan", H, G, N, P)
    g = torch.Generator().manual_seed(H * N)
    with torch.no_grad():
        a.A_log.copy_(rn(g, H, mean=-1.0)), b.A_log.copy_(a.A_log)
    x, Bm, Cm = rn(g, T, H, P).to(dt), rn(g, T, G, N, std=0.5).to(dt), rn(g, T, G, N, std=0.5).to(dt)
    dt_raw, z = rn(g, T, H).to(dt), rn(g, T, H * P).to(dt)
    sa = rn(g, 6, H, N, P)
    sb = sa.clone()
    ya, yb = a(x, Bm, Cm, dt_raw, z, sa), b(x, Bm, Cm, dt_raw, z, sb)
    assert ya.dtype == torch.float32 and rel(ya, yb) < 3e-6 and rel(sa, sb) < 3e-6
    w = rn(g, H * P)
    for groups in (1, H):
        assert rel(hip_layers().group_rms_norm(ya, w, groups, 1e-6, dt), R.group_rms_norm(yb, w, groups, 1e-6, dt)) < tol(dt)


@pytest.mark.parametrize("C,taps", [(96, 4), (100, 2), (1032, 3), (64, 1), (96, 11), (40, 9)])
def test_conv_bias_silu(dt, step, C, taps):
    T, _ = step
    a, b = pair("ConvBiasSilu", C, taps)
    g = torch.Generator().manual_seed(C)
    x = rn(g, T, C + 8).to(dt)[:, 8:]
    sa = rn(g, 6, taps - 1, C).to(dt)
    sb = sa.clone()
    ya, yb = a(x, sa), b(x, sb)
    assert rel(ya, yb) < tol(dt) and torch.equal(sa, sb)


@pytest.mark.parametrize("H,G,D,Dv,chunk,rot", [(6, 3, 10, 8, 7, 6), (4, 1, 40, 56, 12, 40), (2, 2, 64, 64, 20, 32), (4, 2, 128, 64, 0, 64),
                                                 (2, 1, 64, 128, 9, 0), (2, 2, 128, 128, 16, 128), (3, 1, 20, 130, 5, 4), (18, 2, 16, 12, 7, 8), (16, 1, 64, 64, 0, 64)])
def test_chunk_sigmoid_attention(dt, step, H, G, D, Dv, chunk, rot):
    """Head sizes 64 / 128 in bfloat16 take the MFMA tile kernel for the rows of sequences with several rows."""
    T, pos = step
    a, b = pair("ChunkSigmoidAttention", H, G, D, Dv, 1.0 / D ** 0.5, chunk, rot, 300.0, 1e-6)
    g = torch.Generator().manual_seed(D + Dv)
    with torch.no_grad():
        a.head_bias.copy_(rn(g, H, mean=-1.0)), b.head_bias.copy_(a.head_bias)
    q, k, v = rn(g, T, H, D).to(dt), rn(g, T, G, D).to(dt), rn(g, T, G, Dv).to(dt)
    kca, vca = rn(g, 40, 8, G, D).to(dt), rn(g, 40, 8, G, Dv).to(dt)
    kcb, vcb = kca.clone(), vca.clone()
    ya, yb = a(q, k, v, pos, kca, vca), b(q, k, v, pos, kcb, vcb)
    assert rel(kca, kcb) < tol(dt) and rel(vca, vcb) < tol(dt)
    assert rel(ya, yb) < (2e-5 if dt == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("D,Dv,chunk", [(64, 64, 100), (128, 128, 64), (64, 128, 0)])
def test_chunk_sigmoid_attention_long_portions_on_the_tile_kernel(D, Dv, chunk):
    """Portions of several tiles whose chunk edges fall inside tiles, cached keys in front, single rows beside them."""
    dt, H, G = torch.bfloat16, 4, 2
    n_q, n_k = [1, 200, 130, 1, 64], [77, 333, 130, 1, 164]
    ctx, pos = paged_context(n_q, n_k, 16, 60, 3, DEV, slots=[0, 1, 2, 3, 4])
    ctx.cu_seqlens_q_host = np.array([0, 1, 201, 331, 332, 396], dtype=np.int32)
    nv.set_context(ctx)
    try:
        a, b = pair("ChunkSigmoidAttention", H, G, D, Dv, 1.0 / D ** 0.5, chunk, D // 2, 10000.0, 1e-6)
        g = torch.Generator().manual_seed(D * Dv)
        T = sum(n_q)
        q, k, v = rn(g, T, H, D).to(dt), rn(g, T, G, D).to(dt), rn(g, T, G, Dv).to(dt)
        kca, vca = rn(g, 60, 16, G, D).to(dt), rn(g, 60, 16, G, Dv).to(dt)
        kcb, vcb = kca.clone(), vca.clone()
        ya, yb = a(q, k, v, pos, kca, vca), b(q, k, v, pos, kcb, vcb)
        assert rel(ya, yb) < 1.5e-2
        rows = (ya.float() - yb.float()).norm(dim=1) / yb.float().norm(dim=1).clamp_min(1e-3)
        assert rows.max().item() < 5e-2                 # no single row is off (a masked or a missed key would be)
    finally:
        nv.set_context(None)


@pytest.mark.parametrize("E,top,ff,W", [(5, 2, 12, 36), (12, 2, 48, 288), (40, 1, 24, 100), (3, 3, 130, 64)])
def test_table_experts(dt, E, top, ff, W):
    g = torch.Generator().manual_seed(E * ff)
    V, T = 50, 61
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32).to(DEV)
    ids = torch.randint(0, V, (T,), generator=g).to(DEV)
    h = rn(g, T, W).to(dt)
    gu, dn = rn(g, E, 2 * ff, W, std=W ** -0.5).to(dt), rn(g, E, W, ff, std=ff ** -0.5).to(dt)
    ya, yb = hip_layers().TableExperts(top)(h, table, ids, gu, dn), R.TableExperts(top)(h, table, ids, gu, dn)
    assert ya.shape == yb.shape and rel(ya, yb) < (3e-6 if dt == torch.float32 else 1e-2)
