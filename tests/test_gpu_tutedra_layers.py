"""GPU parity of the HIP layers Tutedra is built from against their eager stand-ins (oracle/ref_tutedra_modules.py),
layer by layer, in float32 and bfloat16, on a mixed step (prompt portions beside single rows, shuffled pages, state
slots in any order, states and pages that others left behind) with sizes that exercise the kernels' tails and their
vector paths: widths that are and are not a multiple of a 16-byte piece, head sizes on and off the two-per-lane layout,
odd strides, rotated parts of 2 to 128 dimensions, memories between the register layouts, experts that get no row."""
import pytest
import torch

import nanovllm_amd as nv
from buvalix_util import paged_context
from oracle import ref_tutedra_modules as R

pytestmark = pytest.mark.gpu
DEV = "cuda"


def hip_layers():
    from nanovllm_amd.model.tutedra import _default_layers
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


@pytest.mark.parametrize("W", [96, 100, 2048, 521])
def test_scaled_boundary(dt, W):
    L, g, T = hip_layers(), torch.Generator().manual_seed(W), 9
    x, a1, z, parts = rn(g, T, W), rn(g, T, W).to(dt), rn(g, T, W + 1).to(dt), rn(g, T, 3, W)
    ls, nw = rn(g, W, std=0.3, mean=0.8), rn(g, W, std=0.2, mean=1.0)
    xa, xb = x.clone(), x.clone()
    kw = dict(add=a1, gated=(z[:, :W], z[:, W]), parts=parts, col_scale=ls, norm=nw, eps=1e-6, out_dtype=dt, want_f32=True)
    (a32, a), (b32, b) = L.stream_boundary_scaled(xa, **kw), R.stream_boundary_scaled(xb, **kw)
    assert rel(xa, xb) < 3e-6 and rel(a32, b32) < 3e-6 and rel(a, b) < tol(dt)
    (a32, a), (b32, b) = L.stream_boundary_scaled(xa, norm=nw, eps=1e-6, out_dtype=dt), R.stream_boundary_scaled(xb, norm=nw, eps=1e-6, out_dtype=dt)
    assert a32 is None and rel(xa, xb) < 3e-6 and rel(a, b) < tol(dt)


@pytest.mark.parametrize("cols,stride", [(64, 64), (100, 100), (8192, 8192), (48, 49), (520, 528)])
def test_polynomial_activation(dt, cols, stride):
    a, b = pair("PolyNorm", 1e-6)
    g = torch.Generator().manual_seed(cols)
    z = rn(g, 7, stride, std=2.0).to(dt)[:, :cols]
    assert rel(a(z), b(z)) < tol(dt)


@pytest.mark.parametrize("C,taps", [(96, 3), (100, 4), (24, 1), (72, 11), (3072, 4)])
def test_short_convolution_without_activation(dt, step, C, taps):
    T, _ = step
    a, b = pair("ShortConv", C, taps)
    g = torch.Generator().manual_seed(C)
    x = rn(g, T, C).to(dt)
    sa = rn(g, 6, taps - 1, C).to(dt)
    sb = sa.clone()
    ya, yb = a(x, sa), b(x, sb)
    assert rel(ya, yb) < tol(dt) and (taps == 1 or rel(sa[SLOTS], sb[SLOTS]) < 1e-6)
    assert (ya.float() < 0).any()                       # no activation clipped it


@pytest.mark.parametrize("H,G,D,rot,scaling", [
    (4, 2, 12, 8, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16}), (6, 1, 128, 64, None), (2, 2, 128, 128, None),
    (3, 3, 10, 10, None), (9, 1, 16, 2, None), (2, 1, 160, 32, {"factor": 8.0, "low": 0.5, "high": 2.0, "original": 64}), (4, 4, 7, 0, None)])
def test_key_tied_attention(dt, step, H, G, D, rot, scaling):
    T, pos = step
    a, b = pair("KeyTiedAttention", H, G, D, 1.7 / D ** 0.5, 1e-6, rot, 300.0, scaling)
    g = torch.Generator().manual_seed(H * D)
    qk = rn(g, T, (H + G) * D + 2).to(dt)               # rows of a wider product: an even, unaligned token stride
    q, k = qk[:, :H * D].unflatten(1, (H, D)), qk[:, H * D:(H + G) * D].unflatten(1, (G, D))
    ka, va = rn(g, 40, 8, G, D).to(dt), rn(g, 40, 8, G, D).to(dt)      # stale pages
    kb, vb = ka.clone(), va.clone()
    ya, yb = a(q, k, pos, ka, va), b(q, k, pos, kb, vb)
    assert rel(ya, yb) < tol(dt) and rel(ka, kb) < tol(dt) and torch.equal(va, vb)


@pytest.mark.parametrize("H,Dk,Dv,cap", [(3, 10, 6, 9.0), (2, 64, 64, 15.0), (1, 100, 17, 2.0), (2, 33, 130, 30.0), (1, 256, 200, 12.0)])
def test_matrix_memory(dt, step, H, Dk, Dv, cap):
    T, _ = step
    a, b = pair("MatrixLSTMMemory", H, Dk, Dv, cap, 1e-6)
    g = torch.Generator().manual_seed(Dk)
    q, k, v = (rn(g, T, H, d).to(dt) for d in (Dk, Dk, Dv))
    pre, gate = rn(g, T, 2 * H, std=4.0), rn(g, T, H * Dv).to(dt)
    ca = {n: rn(g, 6, *shape, std=0.5) for n, (shape, _) in a.state_shapes().items()}      # what others left in the slots
    cb = {n: t.clone() for n, t in ca.items()}
    ya, yb = a(q, k, v, pre, gate, ca), b(q, k, v, pre, gate, cb)
    assert rel(ya, yb) < tol(dt)
    for n in ca:
        assert rel(ca[n][SLOTS], cb[n][SLOTS]) < 1e-5, n


@pytest.mark.parametrize("H,Dk,Dv", [(2, 12, 9), (2, 64, 64), (1, 100, 17), (3, 5, 130), (1, 256, 256)])
def test_gated_write_memory(dt, step, H, Dk, Dv):
    T, _ = step
    a, b = pair("GatedWriteMemory", H, Dk, Dv, 1e-6)
    with torch.no_grad():
        for m in (a, b):
            m.lower.copy_(torch.linspace(0.0, 0.99, H * Dk))
    g = torch.Generator().manual_seed(Dk)
    q, f, v = (rn(g, T, H, d).to(dt) for d in (Dk, Dk, Dv))
    ca = {"state": rn(g, 6, H, Dk, Dv, std=0.5)}
    cb = {"state": ca["state"].clone()}
    ya, yb = a(q, f, v, ca), b(q, f, v, cb)
    assert rel(ya, yb) < tol(dt) and rel(ca["state"][SLOTS], cb["state"][SLOTS]) < 1e-5


@pytest.mark.parametrize("E,top,groups,keep", [(8, 2, 4, 2), (6, 6, 1, 1), (9, 1, 9, 4), (64, 6, 8, 3), (130, 8, 2, 1), (512, 16, 16, 4)])
def test_grouped_sigmoid_routing(E, top, groups, keep):
    a, b = pair("GroupedSigmoidRouter", E, top, groups, keep)
    with torch.no_grad():
        for m in (a, b):
            m.correction.sub_(1.0)                      # selection scores below zero
    g = torch.Generator().manual_seed(E)
    logits = rn(g, 77, E, std=2.0)
    (ia, wa), (ib, wb) = a(logits), b(logits)
    assert ia.sort(1).values.tolist() == ib.sort(1).values.tolist() and rel(wa.sort(1).values, wb.sort(1).values) < 1e-6


@pytest.mark.parametrize("T,W,E,top,ff", [(26, 40, 5, 2, 12), (300, 64, 4, 3, 32), (9, 100, 40, 4, 20), (1, 24, 3, 1, 7)])
def test_squared_relu_experts(dt, T, W, E, top, ff):
    a, b = hip_layers().SquaredReluExperts(), R.SquaredReluExperts()
    g = torch.Generator().manual_seed(T)
    h, up, down = rn(g, T, W).to(dt), rn(g, E, ff, W, std=0.3).to(dt), rn(g, E, W, ff, std=0.3).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32).to(DEV)
    w = torch.rand(T, top, generator=g).to(DEV)
    assert rel(a(h, ids, w, up, down), b(h, ids, w, up, down)) < tol(dt)
