"""HIP kernels of the gated parallel-form stacks (gated residual update
fused with the norm, mean of two normed branches, slice norm, exact gelu,
rotation in both pair layouts with the page store, minGRU in its direct and
segment-parallel forms, attention with capped head-mixed scores, the head
gate and windows of the sink-attention kernels incl. the matrix-core path,
the sink of the latent attention kernels) against the fp32 torch reference
of the same op (ops/reference.py), in bf16 and fp32, at sizes that are
neither powers of two nor multiples of the wave size, on column slices of
wider buffers as the runner passes them."""
import pytest
import torch

from bee2bee_amd import ops
from bee2bee_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

if not torch.cuda.is_available():
    pytest.skip("needs a GPU", allow_module_level=True)

from tests.test_hybrid_ops_gpu import DEV, DTYPES, batch_meta, tol  # noqa: E402


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [37, 48, 200, 1024, 4096])
def test_gated_add_rmsnorm(dtype, W):
    torch.manual_seed(0)
    T = 6
    x = torch.randn(T, W, device=DEV) * 3
    wide = (torch.randn(T, 2 * W + 24, device=DEV) * 2).to(dtype)
    g1, g2 = wide[:, 8 : 8 + W], wide[:, 16 + W : 16 + 2 * W]
    y1 = (torch.randn(T, W, device=DEV) * 2).to(dtype)
    y2 = torch.randn(T, W, device=DEV).to(dtype)
    extra = torch.randn(T, W, device=DEV)
    w = torch.rand(W, device=DEV) + 0.5
    cases = [(y1, g1, y2, g2, None, w), (y1, g1, None, None, None, w),
             (y1, g1, y2, g2, extra, w), (None, None, None, None, extra, w),
             (y1, g1, y2, g2, None, None), (None, None, None, None, None, w)]
    for a, ga, b, gb, e, wn in cases:
        r1, r2 = x.clone(), x.clone()
        o1 = ops.gated_add_rmsnorm(r1, a, ga, b, gb, e, wn, 1e-5, dtype)
        o2 = ref.gated_add_rmsnorm(r2, a, ga, b, gb, e, wn, 1e-5, dtype)
        torch.testing.assert_close(r1, r2, rtol=2e-6, atol=4e-6)
        if wn is None:
            assert o1 is None and o2 is None
        else:
            torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [37, 320, 2048])
def test_pair_norm_slice_norm_gelu(dtype, W):
    torch.manual_seed(1)
    a = (torch.randn(5, W, device=DEV) * 3).to(dtype)
    b = (torch.randn(5, W, device=DEV) * 0.2).to(dtype)
    wa, wb = torch.randn(W, device=DEV), torch.randn(W, device=DEV)
    torch.testing.assert_close(
        ops.pair_rmsnorm_mean(a, wa, b, wb, 1e-5, dtype).float(),
        ref.pair_rmsnorm_mean(a, wa, b, wb, 1e-5, dtype).float(), **tol(dtype))
    wide = (torch.randn(9, W + 13, device=DEV) * 2).to(dtype)
    sl = wide[:, 5 : 5 + W]
    o = ops.slice_rmsnorm(sl, wa, 1e-5)
    assert o.is_contiguous() and o.dtype == dtype
    torch.testing.assert_close(o.float(),
                               ref.slice_rmsnorm(sl, wa, 1e-5).float(),
                               **tol(dtype))
    z = (torch.randn(7, W, device=DEV) * 2.5).to(dtype)
    torch.testing.assert_close(ops.gelu_erf(z).float(),
                               ref.gelu_erf(z).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [True, False])
@pytest.mark.parametrize("H,G,D,Dv,dims", [(6, 2, 48, 40, 48), (4, 4, 72, 72, 32),
                                           (3, 1, 200, 17, 0), (8, 2, 128, 128, 64),
                                           (5, 5, 34, 6, 2)])
@pytest.mark.parametrize("conv_out", [False, True])
def test_rope_store(dtype, inter, H, G, D, Dv, dims, conv_out):
    """q in place (inputs of the activation type) and fp32 inputs (as a
    convolution leaves them) into pages of the activation type"""
    torch.manual_seed(1)
    bs, nb = 16, 12
    m = batch_meta([5, 1, 9], [0, 37, 3], bs, nb)
    T = m["T"]
    in_dt = torch.float32 if conv_out else dtype
    proj = (torch.randn(T, (H + G) * D + G * Dv, device=DEV) * 2).to(in_dt)
    sc = {"kind": "banded", "factor": 4.0, "low": 1.0, "high": 4.0,
          "original": 64.0}
    cos, sin = ref.rope_freq_tables(600, dims, 5000.0, sc, DEV) if dims \
        else (None, None)
    outs = []
    for fn in (ops, ref):
        p = proj.clone()
        q = p[:, : H * D].view(T, H, D)
        k = p[:, H * D : (H + G) * D].view(T, G, D)
        v = p[:, (H + G) * D :].view(T, G, Dv)
        q_out = torch.zeros(T, H, D, device=DEV, dtype=dtype) if conv_out else q
        kc = torch.zeros(nb, G, bs, D, device=DEV, dtype=dtype)
        vc = torch.zeros(nb, G, bs, Dv, device=DEV, dtype=dtype)
        fn.rope_store(q, k, v, q_out, dims, inter, m["pos"], cos, sin, 0.37,
                      kc, vc, m["slot_map"])
        outs.append((q_out.clone(), kc, vc))
    for a, b in zip(*outs):
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [7, 224, 1000])
@pytest.mark.parametrize("lens,starts,mq", [
    ([5, 1, 9], [0, 37, 3], 9),            # direct form
    ([300, 1, 130, 64, 2], [0, 5, 77, 0, 9], 300),   # segments + scan
    ([1, 1, 1], [4, 0, 90], 1)])
def test_min_gru(dtype, N, lens, starts, mq):
    torch.manual_seed(2)
    m = batch_meta(lens, starts, 16, 64)
    T = m["T"]
    wide = (torch.randn(T, 3 * N + 16, device=DEV) * 2).to(dtype)
    z, x, g = wide[:, 3 : 3 + N], wide[:, 5 + N : 5 + 2 * N], \
        wide[:, 9 + 2 * N : 9 + 3 * N]
    state = torch.randn(len(lens) + 2, N, device=DEV)
    # a slot whose sequence starts here is not read: poison it
    for b, s in enumerate(starts):
        if s == 0:
            state[int(m["state_slots"][b])] = float("nan")
    s1, s2 = state.clone(), state.clone()
    o1 = torch.zeros(T, N + 3, device=DEV, dtype=dtype)[:, 2 : 2 + N]
    o2 = torch.zeros(T, N, device=DEV, dtype=dtype)
    ops.min_gru(z, x, g, s1, m["state_slots"], m["cu"], m["pos"], o1, mq)
    ref.min_gru(z, x, g, s2, m["state_slots"], m["cu"], m["pos"], o2)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dtype))
    live = m["state_slots"].long()
    torch.testing.assert_close(s1[live], s2[live], rtol=1e-5, atol=1e-5)


def _gqa_case(dtype, lens, starts, H, G, D, Dv, window, bs, softcap, mixed,
              sink, gated, seed=0):
    torch.manual_seed(seed)
    need = sum(-(-(s + L) // bs) for L, s in zip(lens, starts))
    m = batch_meta(lens, starts, bs, need + 3, seed)
    T = m["T"]
    q = (torch.randn(T, H, D, device=DEV) * (2.0 if softcap else 1.0)).to(dtype)
    kc = torch.randn(need + 3, G, bs, D, device=DEV).to(dtype)
    vc = torch.randn(need + 3, G, bs, Dv, device=DEV).to(dtype)
    talk = (torch.eye(H, device=DEV) + 0.3 * torch.randn(H, H, device=DEV)) \
        if mixed else None
    sk = {"zero": torch.zeros(H, device=DEV),
          "learned": torch.randn(H, device=DEV) * 2, "none": None}[sink]
    wide = torch.randn(T, H + 16, device=DEV).to(dtype)
    hg = wide[:, 8 : 8 + H] if gated else None
    o1 = torch.zeros(T, H * Dv, device=DEV, dtype=dtype)
    o2 = torch.zeros(T, H * Dv, device=DEV, dtype=torch.float32)
    ops.gqa_attn(q, kc, vc, m["bt"], m["pos"], m["seq"], m["cu"], softcap,
                 talk, sk, hg, window, o1, max(lens))
    ref.gqa_attn(q.float(), kc.float(), vc.float(), m["bt"], m["pos"],
                 m["seq"], m["cu"], softcap, talk, sk,
                 None if hg is None else hg.float(), window, o2)
    return o1.float(), o2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,window", [
    (8, 2, 56, 72, 90), (6, 3, 40, 24, 0), (4, 4, 72, 130, 7),
    (5, 1, 33, 17, 20), (16, 8, 64, 64, 50), (12, 6, 16, 200, 1)])
@pytest.mark.parametrize("softcap,sink,gated", [(3.0, "zero", False),
                                                (0.0, "learned", True),
                                                (1.5, "none", True)])
def test_mixed_score_attention(dtype, H, G, D, Dv, window, softcap, sink,
                               gated):
    """prompt portions, single rows and a row far into its sequence in one
    step; scattered pages; windows smaller and larger than the history"""
    a, b = _gqa_case(dtype, [5, 1, 33, 1, 2], [0, 120, 17, 0, 300], H, G, D,
                     Dv, window, 16, softcap, True, sink, gated)
    t = tol(dtype)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_score_attention_decode_splits(dtype):
    """few rows with long histories: the keys are split over waves and the
    partials merged with the sink and the gate"""
    t = tol(dtype)
    a, b = _gqa_case(dtype, [1, 1, 1], [700, 64, 1300], 8, 2, 64, 64, 0, 64,
                     4.0, True, "zero", True)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)
    a, b = _gqa_case(dtype, [1, 1], [700, 2000], 8, 4, 128, 128, 512, 256,
                     0.0, True, "learned", False)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,window", [
    (8, 2, 56, 72, 90), (6, 3, 40, 24, 0), (4, 4, 64, 128, 7),
    (5, 1, 33, 17, 20)])
@pytest.mark.parametrize("sink,gated", [("none", True), ("zero", True),
                                        ("learned", False)])
def test_plain_attention_gate_window(dtype, H, G, D, Dv, window, sink, gated):
    """no cap and no mix: the sink-attention kernels with a head gate"""
    a, b = _gqa_case(dtype, [5, 1, 33, 1, 2], [0, 120, 17, 0, 300], H, G, D,
                     Dv, window, 16, 0.0, False, sink, gated)
    t = tol(dtype)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)
    a, b = _gqa_case(dtype, [1, 1, 1], [700, 64, 1300], H, G, D, Dv, window,
                     64, 0.0, False, sink, gated)
    torch.testing.assert_close(a, b, rtol=t["rtol"], atol=t["atol"] * 3)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G,window", [(1, 0), (2, 100), (4, 64), (2, 1),
                                      (3, 300), (2, 40), (2, 65)])
@pytest.mark.parametrize("sink,gated", [("none", True), ("zero", False)])
def test_plain_attention_matrix_core_windows(D, G, window, sink, gated):
    """bf16 prompt portions of head size 64/128: the query-tiled kernel with
    windows that end inside, at and before a key tile, chunks with history,
    a chunk shorter than a tile, single rows riding along"""
    a, b = _gqa_case(torch.bfloat16, [70, 1, 130, 16, 1],
                     [0, 200, 57, 500, 0], 2 * G, G, D, D, window, 32, 0.0,
                     False, sink, gated, seed=3)
    torch.testing.assert_close(a, b, rtol=2e-2, atol=4e-2)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G,window", [(1, 0), (2, 100), (4, 64), (2, 1),
                                      (3, 300), (2, 40), (2, 65)])
@pytest.mark.parametrize("softcap,sink,gated", [(3.0, "zero", False),
                                                (0.0, "learned", True)])
def test_mixed_score_attention_matrix_core(D, G, window, softcap, sink, gated):
    """bf16 prompt portions of head size 64/128: tile scores on the matrix
    cores, the head mix on the score buffer, softmax and P V from the mixed
    tiles; windows that end inside, at and before a key tile, chunks with
    history, a chunk shorter than a tile, single rows riding along"""
    a, b = _gqa_case(torch.bfloat16, [70, 1, 130, 16, 1],
                     [0, 200, 57, 500, 0], 2 * G, G, D, D, window, 32,
                     softcap, True, sink, gated, seed=3)
    torch.testing.assert_close(a, b, rtol=2e-2, atol=4e-2)


def test_mixed_score_attention_matrix_core_many_tiles():
    """a long portion cut into several launches of the score buffer"""
    a, b = _gqa_case(torch.bfloat16, [700, 300], [100, 0], 8, 2, 64, 64, 0,
                     64, 2.0, True, "zero", False, seed=4)
    torch.testing.assert_close(a, b, rtol=2e-2, atol=4e-2)


def _latent_case(dtype, lens, starts, H, C, R, window, sink, bs=16, seed=3):
    torch.manual_seed(seed)
    need = sum(-(-(s + L) // bs) for L, s in zip(lens, starts))
    m = batch_meta(lens, starts, bs, need + 2, seed)
    T = m["T"]
    cache = torch.randn(need + 2, bs, C + R, device=DEV).to(dtype)
    q_abs = (torch.randn(H, T, C, device=DEV) * C ** -0.5).to(dtype)
    q_rot = torch.randn(T, H, R, device=DEV).to(dtype)
    gate = torch.randn(T, H, device=DEV).to(dtype)
    sk = torch.randn(H, device=DEV) * 2 if sink else None
    o1 = ops.latent_attn(q_abs, q_rot, gate, cache, m["bt"], m["pos"],
                         m["seq"], m["cu"], window, 0.3, max(lens), sink=sk)
    o2 = ref.latent_attn(q_abs, q_rot, gate, cache, m["bt"], m["pos"],
                         m["seq"], m["cu"], window, 0.3, sink=sk)
    return o1.float(), o2.float()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,C,R", [(4, 32, 8), (8, 64, 32), (3, 72, 10),
                                   (16, 128, 64)])
@pytest.mark.parametrize("window", [0, 9])
@pytest.mark.parametrize("sink", [True, False])
def test_latent_attention_sink(dtype, H, C, R, window, sink):
    """mixed steps (generic kernel), prompt portions (matrix cores in bf16)
    and decode steps with key splits, with and without the sink, with a
    window and without one"""
    for lens, starts in (([33, 1, 2, 1], [0, 47, 15, 0]),
                         ([40, 17], [0, 30]),
                         ([1, 1, 1, 1, 1], [0, 47, 15, 200, 95])):
        a, b = _latent_case(dtype, lens, starts, H, C, R, window, sink)
        torch.testing.assert_close(a, b, **tol(dtype))


@pytest.mark.parametrize("score", ["sigmoid", "softmax"])
@pytest.mark.parametrize("E,top,n_groups,keep,group_top", [
    (8, 3, 4, 3, 2), (8, 2, 2, 1, 2), (6, 1, 3, 2, 1), (4, 4, 1, 1, 1),
    (9, 2, 9, 4, 1), (12, 3, 3, 3, 2), (64, 8, 8, 4, 2), (128, 6, 16, 3, 3)])
def test_group_topk_gate(score, E, top, n_groups, keep, group_top):
    """the routing kernel against the torch-op reference: same experts,
    same weights (random logits have no ties)"""
    torch.manual_seed(9)
    logits = torch.randn(333, E, device=DEV) * 2
    w1, i1 = ops.group_topk_gate(logits, top, n_groups, keep, score, group_top)
    w2, i2 = ref.group_topk_gate(logits, top, n_groups, keep, score, group_top)
    assert i1.dtype == torch.int32 and w1.dtype == torch.float32
    o1, o2 = i1.long().sort(1), i2.long().sort(1)
    assert torch.equal(o1.values, o2.values)
    torch.testing.assert_close(w1.gather(1, o1.indices),
                               w2.gather(1, o2.indices), rtol=1e-5, atol=1e-6)
