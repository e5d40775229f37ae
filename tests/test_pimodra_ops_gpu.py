"""HIP kernels of the weighted-sandwich stacks (grouped norm fused with the
residual and step add, rotate-then-unit-norm page store, head-mixing
windowed attention in its generic and matrix-core forms, PolyNorm, silu GLU)
against the fp32 torch reference of the same op (ops/reference.py), in bf16
and fp32, at sizes that are neither powers of two nor multiples of the wave
size, on column slices of wider buffers as the runner passes them."""
import pytest
import torch

from bee2bee_amd import ops
from bee2bee_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

if not torch.cuda.is_available():
    pytest.skip("needs a GPU", allow_module_level=True)

from tests.test_hybrid_ops_gpu import DEV, DTYPES, batch_meta, tol  # noqa: E402


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,groups", [(36, 3), (48, 1), (200, 4), (1024, 2),
                                      (4096, 8)])
def test_group_norms(dtype, W, groups):
    torch.manual_seed(0)
    x = torch.randn(6, W, device=DEV) * 3
    w1, w2 = torch.randn(W, device=DEV), torch.randn(W, device=DEV)
    step = torch.randn(W, device=DEV)
    y = (torch.randn(6, W, device=DEV) * 2).to(dtype)
    cases = [(None, None, None, w2), (y, w1, None, w2), (y, w1, step, w2),
             (None, None, step, w2), (y, w1, None, None), (y, w1, step, None)]
    for yy, wp, st, wn in cases:
        r1, r2 = x.clone(), x.clone()
        a = ops.add_group_rmsnorm(r1, yy, wp, st, wn, groups, 1e-5, dtype)
        b = ref.add_group_rmsnorm(r2, yy, wp, st, wn, groups, 1e-5, dtype)
        torch.testing.assert_close(r1, r2, rtol=2e-6, atol=2e-6)
        if wn is None:
            assert a is None and b is None
        else:
            torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


def _tables(dims, scaling, n=600):
    return ref.rope_tables_scaled(n, dims, 5000.0, scaling, DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,dims", [(6, 2, 48, 40, 48), (4, 4, 72, 72, 32),
                                           (3, 1, 200, 17, 0), (8, 2, 128, 128, 128)])
def test_rope_unit_store(dtype, H, G, D, Dv, dims):
    torch.manual_seed(1)
    bs, nb = 16, 12
    m = batch_meta([5, 1, 9], [0, 37, 3], bs, nb)
    T = m["T"]
    proj = (torch.randn(T, H * D + G * D + G * Dv + 8, device=DEV) * 2).to(dtype)
    sc = {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0}
    cos, sin = _tables(dims, sc) if dims else (None, None)
    outs = []
    for fn in (ops, ref):
        p = proj.clone()
        q = p[:, : H * D].view(T, H, D)
        k = p[:, H * D : (H + G) * D].view(T, G, D)
        v = p[:, (H + G) * D : (H + G) * D + G * Dv].view(T, G, Dv)
        kc = torch.zeros(nb, G, bs, D, device=DEV, dtype=dtype)
        vc = torch.zeros(nb, G, bs, Dv, device=DEV, dtype=dtype)
        fn.rope_unit_store(q, k, v, 1e-6, dims, m["pos"], cos, sin, 0.37, kc,
                           vc, m["slot_map"])
        outs.append((p, kc, vc))
    for a, b in zip(*outs):
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


def _attn_case(dtype, lens, starts, H, G, D, Dv, window, bs, seed=0,
               path="auto"):
    torch.manual_seed(seed)
    need = sum(-(-(s + L) // bs) for L, s in zip(lens, starts))
    m = batch_meta(lens, starts, bs, need + 3, seed)
    T = m["T"]
    q = torch.randn(T, H, D, device=DEV).to(dtype)
    nbk = need + 3
    kc = (torch.randn(nbk, G, bs, D, device=DEV)).to(dtype)
    vc = (torch.randn(nbk, G, bs, Dv, device=DEV)).to(dtype)
    talk = torch.eye(H, device=DEV) + 0.3 * torch.randn(H, H, device=DEV)
    wide = torch.randn(T, H * Dv + 16, device=DEV).to(dtype)
    gate = wide[:, 8 : 8 + H * Dv]
    o1 = torch.zeros(T, H * Dv, device=DEV, dtype=dtype)
    o2 = torch.zeros_like(o1)
    mq = max(lens)
    ops.talk_attn(q, kc, vc, m["bt"], m["pos"], m["seq"], m["cu"], talk, gate,
                  window, o1, mq, path)
    ref.talk_attn(q.float(), kc.float(), vc.float(), m["bt"], m["pos"],
                  m["seq"], m["cu"], talk, gate.float(), window, o2)
    return o1.float(), o2.float()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,window", [
    (8, 2, 56, 72, 90), (6, 3, 40, 24, 0), (4, 4, 72, 130, 7),
    (5, 1, 33, 17, 20), (16, 8, 64, 64, 50), (12, 6, 16, 200, 1)])
@pytest.mark.parametrize("path", ["scored", "cross"])
def test_talk_attn_generic(dtype, H, G, D, Dv, window, path):
    """prompt portions, single rows and a row far into its sequence in one
    step; pages scattered; windows smaller and larger than the history;
    both generic forms (heads mixed before / after the values)"""
    a, b = _attn_case(dtype, [5, 1, 33, 1, 2], [0, 120, 17, 0, 300], H, G, D,
                      Dv, window, 16, path=path)
    t = tol(dtype)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("path", ["scored", "cross"])
def test_talk_attn_decode_splits(dtype, path):
    """few rows with long histories: the keys are split over waves"""
    a, b = _attn_case(dtype, [1, 1, 1], [700, 64, 1300], 8, 2, 64, 64, 0, 64,
                      path=path)
    t = tol(dtype)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)
    a, b = _attn_case(dtype, [1, 1], [700, 2000], 8, 4, 128, 128, 512, 256,
                      path=path)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G,window", [(1, 0), (2, 100), (4, 64), (2, 1),
                                      (3, 300), (8, 40), (6, 0)])
def test_talk_attn_matrix_core(D, G, window):
    """bf16 prompt portions of head size 64/128: the query-tiled kernel;
    chunks with history, a chunk shorter than a tile, single rows riding
    along, windows that end inside, at and before a key tile"""
    H = G * 2
    a, b = _attn_case(torch.bfloat16, [70, 1, 130, 16, 1],
                      [0, 200, 57, 500, 0], H, G, D, D, window, 32, seed=3)
    torch.testing.assert_close(a, b, rtol=2e-2, atol=4e-2)


def test_talk_attn_matrix_core_weights_32bit():
    """the matrix-core path carries softmax weights with more than bf16
    precision: with values that are exact in bf16 and one dominant key
    the output error stays far below a bf16 rounding of the weights"""
    torch.manual_seed(5)
    H, G, D, bs = 4, 2, 64, 32
    a, b = _attn_case(torch.bfloat16, [64], [0], H, G, D, D, 0, bs, seed=7)
    # outputs are rounded to bf16 once at the end: relative error ~2^-9
    err = (a - b).abs().max() / b.abs().max()
    assert err < 6e-3, err


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [24, 100, 384, 8192])
def test_polynorm(dtype, N):
    torch.manual_seed(2)
    z = (torch.randn(7, N, device=DEV) * 1.5).to(dtype)
    coef = torch.tensor([0.4, -0.3, 0.2, 0.05], device=DEV)
    a = ops.polynorm(z, coef, 1e-6, dtype)
    b = ref.polynorm(z, coef, 1e-6, dtype)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("I", [24, 37, 1024])
def test_silu_glu(dtype, I):
    torch.manual_seed(3)
    gu = (torch.randn(9, 2 * I, device=DEV) * 2).to(dtype)
    torch.testing.assert_close(ops.silu_glu(gu).float(),
                               ref.silu_glu(gu).float(), **tol(dtype))
