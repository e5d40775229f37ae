"""Zevilorn on the CPU reference path against the plain oracle
(tests/zevilorn_oracle.py): each mechanism alone, then the served model —
whole prompts, decoding, portions, mixed batches with page and slot reuse,
window and page edges, the scheduler's own greedy generation."""
import io
import json
import math
import sys

import pytest
import torch

from bee2bee_amd.models.spec import zevilorn_spec
from bee2bee_amd.ops import reference as ref
from tests import zevilorn_oracle as O
from tests.zevilorn_util import (assert_logits, chunk_schedule, make_engine,
                                 oracle_logits, random_tokens, rel_err, replay)

F32, F64 = torch.float32, torch.float64


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


def pages(lens, starts, bs, seed=0):
    """Packed-chunk metadata with scattered pages."""
    g = torch.Generator().manual_seed(seed)
    need = [-(-(s + L) // bs) for L, s in zip(lens, starts)]
    nb = sum(need) + 2
    perm = torch.randperm(nb, generator=g).tolist()
    bt = torch.zeros(len(lens), max(need), dtype=torch.int32)
    k = 0
    for b in range(len(lens)):
        for j in range(need[b]):
            bt[b, j] = perm[k]
            k += 1
    cu, pos, seq = [0], [], []
    for b, (L, s) in enumerate(zip(lens, starts)):
        cu.append(cu[-1] + L)
        pos += list(range(s, s + L))
        seq += [b] * L
    slot = [int(bt[b, p // bs]) * bs + p % bs for b, p in zip(seq, pos)]
    return dict(cu=i32(cu), pos=i32(pos), seq=i32(seq), bt=bt, slot=i32(slot),
                nb=nb, T=cu[-1])


# ----------------------------------------------------------- mechanisms

@pytest.mark.parametrize("W", [5, 24])
def test_gated_residual_update(W):
    torch.manual_seed(0)
    x = torch.randn(4, W) * 3
    y1, y2 = torch.randn(4, W), torch.randn(4, W) * 2
    g1, g2 = torch.randn(4, W) * 2, torch.randn(4, W)
    e, w = torch.randn(4, W), torch.randn(W)
    want_x = (x.double() + O.sigmoid(g1.double()) * y1.double()
              + O.sigmoid(g2.double()) * y2.double() + e.double())
    want = O.unit(want_x, 1e-5) * w.double()
    r = x.clone()
    got = ref.gated_add_rmsnorm(r, y1, g1, y2, g2, e, w, 1e-5, F32)
    assert torch.allclose(r.double(), want_x, atol=1e-5)
    assert torch.allclose(got.double(), want, atol=1e-5)
    # one sublayer, nothing to add, nothing to return
    r = x.clone()
    assert ref.gated_add_rmsnorm(r, y1, g1, None, None, None, None, 1e-5,
                                 F32) is None
    assert torch.allclose(r.double(), x.double() + O.sigmoid(g1.double())
                          * y1.double(), atol=1e-5)
    # a closed gate (very negative) shuts the sublayer out
    r = x.clone()
    ref.gated_add_rmsnorm(r, y1 * 1e3, torch.full_like(g1, -60.0), None, None,
                          None, None, 1e-5, F32)
    assert torch.allclose(r, x, atol=1e-6)


@pytest.mark.parametrize("scaling,rule", [
    (None, "none"), ({"factor": 2.0}, "linear"),
    ({"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16}, "banded"),
    ({"factor": 8.0, "low": 2.0, "high": 3.0, "original": 100}, "banded"),
    ({"factor": 3.0, "low": 1.0, "high": 4.0, "original": 4096}, "banded")])
@pytest.mark.parametrize("dims,base", [(4, 100.0), (16, 1e4), (64, 1e6)])
def test_rotation_frequencies(scaling, rule, dims, base):
    from bee2bee_amd.models.hybrid import _rot_scaling

    rot = {"dims": dims, "base": base, "scaling": scaling}
    f = O.frequencies(rot, rule)
    cos, sin = ref.rope_freq_tables(50, dims, base, _rot_scaling(scaling),
                                    "cpu")
    for p in (0, 1, 17, 49):
        for i in range(dims // 2):
            assert abs(float(cos[p, i]) - math.cos(p * f[i])) < 1e-6
            assert abs(float(sin[p, i]) - math.sin(p * f[i])) < 1e-6
    if rule == "banded":
        # the three bands exist in the larger tables: kept, slowed, between
        plain = O.frequencies({"dims": dims, "base": base}, "none")
        ratio = [a / b for a, b in zip(f, plain)]
        assert max(ratio) <= 1.0 + 1e-12
        assert min(ratio) >= 1.0 / scaling["factor"] - 1e-12


@pytest.mark.parametrize("inter", [True, False])
@pytest.mark.parametrize("dims", [0, 2, 6, 8])
def test_rotation_layouts_and_store(inter, dims):
    """both pair layouts, partial rotation, q scaled, k and v to scattered
    pages; rows of other slots untouched"""
    torch.manual_seed(1)
    H, G, D, Dv, bs = 3, 1, 8, 5, 4
    m = pages([5, 2], [3, 0], bs)
    T = m["T"]
    q, k = torch.randn(T, H, D), torch.randn(T, G, D)
    v = torch.randn(T, G, Dv)
    f = [50.0 ** (-2.0 * i / dims) for i in range(dims // 2)] if dims else []
    cos, sin = (ref.rope_freq_tables(20, dims, 50.0, None, "cpu")
                if dims else (None, None))
    kc = torch.full((m["nb"], G, bs, D), float("nan"))
    vc = torch.full((m["nb"], G, bs, Dv), float("nan"))
    q_out = torch.empty_like(q)
    ref.rope_store(q, k, v, q_out, dims, inter, m["pos"], cos, sin, 0.7, kc,
                   vc, m["slot"])
    lay = "interleaved" if inter else "half"
    for b, (lo, hi, start) in enumerate([(0, 5, 3), (5, 7, 0)]):
        pad = torch.zeros(start, H, D, dtype=F64)
        want_q = O.rotate(torch.cat([pad, q[lo:hi].double()]), f, lay)[start:]
        assert torch.allclose(q_out[lo:hi].double(), want_q * 0.7, atol=1e-5)
        padk = torch.zeros(start, G, D, dtype=F64)
        want_k = O.rotate(torch.cat([padk, k[lo:hi].double()]), f, lay)[start:]
        for t in range(lo, hi):
            s = int(m["slot"][t])
            assert torch.allclose(kc[s // bs, :, s % bs].double(),
                                  want_k[t - lo], atol=1e-5)
            assert torch.equal(vc[s // bs, :, s % bs], v[t])
    assert int(torch.isnan(kc[:, 0, :, 0]).sum()) == m["nb"] * bs - T


def _attention_vs_oracle(H, G, D, Dv, window, softcap, mixed, sink, gated,
                         lens_sched, bs=4, seed=0, scale_q=None):
    """One sequence fed in portions through rope_store + gqa_attn over
    NaN-filled scattered pages, against the oracle's whole-sequence math."""
    torch.manual_seed(seed)
    T = sum(lens_sched)
    q, k = torch.randn(T, H, D), torch.randn(T, G, D)
    v = torch.randn(T, G, Dv)
    if scale_q is not None:
        scale_q(q, k)
    talk = torch.eye(H) + 0.4 * torch.randn(H, H) if mixed else None
    sk = {"zero": torch.zeros(H), "learned": torch.randn(H) * 2,
          "none": None}[sink]
    hg = torch.randn(T, H) if gated else None
    s = O.gqa_scores(q.double(), k.double(), 0.5)
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    if mixed:
        s = torch.einsum("hg,gij->hij", talk.double(), s)
    pr = O.softmax_rows(s, O.visible(T, window or None),
                        None if sk is None else sk.double())
    want = O.gqa_apply(pr, v.double()).view(T, H, Dv)
    if gated:
        want = want * O.sigmoid(hg.double())[..., None]
    m = pages([T], [0], bs, seed)
    kc = torch.full((m["nb"], G, bs, D), float("nan"))
    vc = torch.full((m["nb"], G, bs, Dv), float("nan"))
    got = torch.zeros(T, H * Dv)
    at = 0
    for n in lens_sched:
        pos = i32(list(range(at, at + n)))
        slot = m["slot"][at:at + n]
        qo = torch.empty(n, H, D)
        ref.rope_store(q[at:at + n], k[at:at + n], v[at:at + n], qo, 0, True,
                       pos, None, None, 0.5, kc, vc, slot)
        out = torch.zeros(n, H * Dv)
        ref.gqa_attn(qo, kc, vc, m["bt"], pos, i32([0] * n), i32([0, n]),
                     softcap, talk, sk, None if hg is None else hg[at:at + n],
                     window, out)
        got[at:at + n] = out
        at += n
    return got.view(T, H, Dv).double(), want, pr


@pytest.mark.parametrize("H,G,D,Dv,window", [(4, 2, 6, 5, 7), (3, 3, 4, 4, 0),
                                             (6, 1, 5, 9, 1), (2, 1, 8, 3, 30)])
@pytest.mark.parametrize("softcap,mixed,sink,gated", [
    (2.0, True, "zero", False), (0.0, False, "none", True),
    (0.0, True, "learned", True), (1.0, False, "zero", False)])
@pytest.mark.parametrize("sched", [[23], [1] * 23, [2, 5, 1, 13, 2],
                                   [2] * 11 + [1]])
def test_attention_options_in_portions(H, G, D, Dv, window, softcap, mixed,
                                       sink, gated, sched):
    got, want, _ = _attention_vs_oracle(H, G, D, Dv, window, softcap, mixed,
                                        sink, gated, sched)
    assert torch.allclose(got, want, atol=2e-5)


def test_zero_sink_takes_its_share():
    """with every score at zero, n visible keys and the zero-logit sink
    share the weight: each key gets 1 / (n + 1), not 1 / n"""
    H, G, D, Dv = 2, 1, 4, 3
    zero = lambda q, k: (q.zero_(), k.zero_())  # noqa: E731
    got, want, pr = _attention_vs_oracle(H, G, D, Dv, 0, 0.0, False, "zero",
                                         False, [6], scale_q=zero)
    assert torch.allclose(got, want, atol=1e-6)
    for i in range(6):
        assert abs(float(pr[0, i, 0]) - 1.0 / (i + 2)) < 1e-12
    # ... and without the sink the weights sum to one
    _, _, pr = _attention_vs_oracle(H, G, D, Dv, 0, 0.0, False, "none", False,
                                    [6], scale_q=zero)
    assert abs(float(pr[0, 5].sum()) - 1.0) < 1e-12


def test_cap_comes_before_the_mix_and_the_mix_before_the_softmax():
    """a huge score is held at the cap; a mix that swaps two heads makes
    each use the OTHER head's scores with its OWN values"""
    torch.manual_seed(3)
    H, G, D, Dv, T = 2, 2, 4, 3, 9
    q, k = torch.randn(T, H, D) * 30, torch.randn(T, G, D)
    v = torch.randn(T, G, Dv)
    m = pages([T], [0], 4)
    kc = torch.zeros(m["nb"], G, 4, D)
    vc = torch.zeros(m["nb"], G, 4, Dv)
    qo = torch.empty_like(q)
    ref.rope_store(q, k, v, qo, 0, True, m["pos"], None, None, 1.0, kc, vc,
                   m["slot"])
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    a, b = torch.zeros(T, H * Dv), torch.zeros(T, H * Dv)
    args = (kc, vc, m["bt"], m["pos"], m["seq"], m["cu"])
    ref.gqa_attn(qo, *args, 1.5, swap, None, None, 0, a)
    s = 1.5 * torch.tanh(O.gqa_scores(q.double(), k.double(), 1.0) / 1.5)
    assert float(s.abs().max()) <= 1.5
    pr = O.softmax_rows(s.flip(0), O.visible(T, None), None)
    want = O.gqa_apply(pr, v.double())
    assert torch.allclose(a.double(), want, atol=1e-5)
    # mixing after the softmax would give something else
    ref.gqa_attn(qo, *args, 1.5, None, None, None, 0, b)
    assert not torch.allclose(a, b.view(T, H, Dv).flip(1).reshape(T, -1),
                              atol=1e-3)


@pytest.mark.parametrize("window", [1, 5, 16, 17])
@pytest.mark.parametrize("sched", [[40], [24] + [1] * 16])
def test_dominant_key_just_inside_and_outside_the_window(window, sched):
    """one far key made dominant: rows that still see it return (almost)
    its value, the first row past the window does not — in prompts and in
    decoding, across page borders (pages of 4)"""
    H, G, D, Dv, T, j = 2, 1, 8, 4, 40, 11

    def plant(q, k):
        k.mul_(0.05)
        q.mul_(0.05)
        k[j, 0, 0] = 30.0
        q[:, :, 0] = 30.0

    got, want, pr = _attention_vs_oracle(H, G, D, Dv, window, 0.0, False,
                                         "zero", False, sched, scale_q=plant)
    assert torch.allclose(got, want, atol=2e-5)
    inside, outside = j + window - 1, j + window
    assert float(pr[0, inside, j]) > 0.99
    assert float(pr[0, outside, j]) == 0.0
    assert float((got[inside] - got[outside]).abs().max()) > 0.05 or window == 1


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_conv_on_projections_over_portions(taps):
    """the conv the attention applies to q|k|v: tap-major weights, carried
    rows per slot, zeros before the start, unequal chunks in one batch"""
    torch.manual_seed(4)
    C = 7
    w = torch.randn(C, taps)
    a, b = torch.randn(11, C), torch.randn(6, C)
    want_a = O.short_conv(a.double(), w.double())
    want_b = O.short_conv(b.double(), w.double())
    state = torch.full((3, max(taps - 1, 0), C), float("nan"))
    wt = w.t().contiguous()
    slots = i32([2, 0])
    got_a, got_b = [], []
    for (la, lb, pa, pb) in [(4, 1, 0, 0), (1, 3, 4, 1), (6, 2, 5, 4)]:
        x = torch.cat([a[pa:pa + la], b[pb:pb + lb]])
        pos = i32(list(range(pa, pa + la)) + list(range(pb, pb + lb)))
        y = ref.short_conv(x, wt, state, slots, i32([0, la, la + lb]),
                           i32([0] * la + [1] * lb), pos, False)
        got_a.append(y[:la])
        got_b.append(y[la:])
    assert torch.allclose(torch.cat(got_a).double(), want_a, atol=1e-5)
    assert torch.allclose(torch.cat(got_b).double(), want_b, atol=1e-5)


@pytest.mark.parametrize("sink", [True, False])
@pytest.mark.parametrize("sched", [[19], [1] * 19, [2, 9, 1, 7]])
def test_latent_attention_with_sink_in_portions(sink, sched):
    """the absorbed form over the paged latent rows against plain per-head
    keys and values; no window; a learned sink logit per head"""
    torch.manual_seed(5)
    H, D, R, Dv, C, T, bs = 3, 6, 4, 5, 7, 19, 4
    qn, qr = torch.randn(T, H, D), torch.randn(T, H, R)
    lat, kr = torch.randn(T, C), torch.randn(T, R)
    w_uk, w_uv = torch.randn(H, D, C), torch.randn(H, C, Dv)
    gate = torch.randn(T, H)
    sk = torch.randn(H) * 2 if sink else None
    f = [300.0 ** (-2.0 * i / R) for i in range(R // 2)]
    # the store norms the latent (unit weight, eps 0): c = lat / rms(lat)
    c = lat.double() / lat.double().pow(2).mean(-1, keepdim=True).sqrt()
    kn = torch.einsum("hdc,tc->thd", w_uk.double(), c)
    vv = torch.einsum("hcv,tc->thv", w_uv.double(), c)
    s = torch.einsum("ihd,jhd->hij", qn.double(), kn)
    s = s + torch.einsum("ihr,jr->hij", O.rotate(qr.double(), f, "half"),
                         O.rotate(kr.double()[:, None], f, "half")[:, 0])
    pr = O.softmax_rows(s * 0.3, O.visible(T, None),
                        None if sk is None else sk.double())
    want = torch.einsum("hij,jhd->ihd", pr, vv) * \
        O.sigmoid(gate.double())[..., None]
    m = pages([T], [0], bs)
    cache = torch.full((m["nb"], bs, C + R), float("nan"))
    cos, sin = ref.rope_freq_tables(32, R, 300.0, None, "cpu")
    got = torch.zeros(T, H, Dv)
    at = 0
    for n in sched:
        pos = i32(list(range(at, at + n)))
        q_rot = qr[at:at + n].clone()
        kv = torch.cat([lat[at:at + n], kr[at:at + n]], -1)
        ref.latent_rope_store(q_rot, kv, torch.ones(C), 0.0, C, R, pos, cos,
                              sin, cache, m["slot"][at:at + n])
        q_abs = torch.bmm(qn[at:at + n].transpose(0, 1), w_uk)
        o = ref.latent_attn(q_abs, q_rot, gate[at:at + n], cache, m["bt"],
                            pos, i32([0] * n), i32([0, n]), 0, 0.3, sink=sk)
        got[at:at + n] = torch.bmm(o, w_uv).transpose(0, 1)
        at += n
    assert torch.allclose(got.double(), want, atol=3e-5)


@pytest.mark.parametrize("j", [0, 15, 16, 17, 131])
@pytest.mark.parametrize("sched", [[300], [280] + [1] * 20])
def test_latent_far_key_among_hundreds(j, sched):
    """no window: one key far back — the first token, both sides of a page
    border — dominates among 300; every later row returns its latent row,
    in a prompt and in decoding, whatever the sink holds"""
    torch.manual_seed(9)
    H, C, R, T, bs = 2, 6, 2, 300, 16
    lat = torch.randn(T, C) * 0.05
    lat[j] = torch.tensor([4.0, -3.0, 2.0, 1.0, -2.0, 3.0])
    m = pages([T], [0], bs)
    cache = torch.full((m["nb"], bs, C + R), float("nan"))
    flat = cache.view(-1, C + R)
    flat[m["slot"].long()] = torch.cat([lat, torch.zeros(T, R)], -1)
    # every query points along the planted row
    q_abs = (lat[j] * 3.0).expand(H, T, C).contiguous()
    q_rot = torch.zeros(T, H, R)
    gate = torch.full((T, H), 40.0)
    sk = torch.tensor([1.0, -2.0])
    got, at = [], 0
    for n in sched:
        pos = i32(list(range(at, at + n)))
        got.append(ref.latent_attn(q_abs[:, at:at + n].contiguous(),
                                   q_rot[at:at + n], gate[at:at + n], cache,
                                   m["bt"], pos, i32([0] * n), i32([0, n]), 0,
                                   1.0, sink=sk))
        at += n
    got = torch.cat(got, 1)
    for t in (max(j, 1), j + 1, 299):
        if t >= j:
            assert torch.allclose(got[:, t], lat[j].expand(H, C), atol=1e-3), t
    if j > 0:       # rows before it do not see it
        assert float(got[:, j - 1].abs().max()) < 1.0


def test_latent_sink_is_not_scaled_and_counts_once():
    """all scores equal: the sink's share is e^sink / (e^sink + n e^s)"""
    H, C, R, T = 2, 3, 2, 5
    cache = torch.zeros(3, 4, C + R)
    m = pages([T], [0], 4)
    q_abs, q_rot = torch.zeros(H, T, C), torch.zeros(T, H, R)
    cache[..., 0] = 1.0
    sk = torch.tensor([0.7, -1.2])
    gate = torch.full((T, H), 40.0)                 # open gate
    o = ref.latent_attn(q_abs, q_rot, gate, cache, m["bt"], m["pos"],
                        m["seq"], m["cu"], 0, 123.0, sink=sk)
    for h in range(H):
        for t in range(T):
            share = (t + 1) / (t + 1 + math.exp(float(sk[h])))
            assert abs(float(o[h, t, 0]) - share) < 1e-6


@pytest.mark.parametrize("N", [1, 13])
@pytest.mark.parametrize("sched", [[31], [1] * 31, [2, 7, 1, 19, 2]])
def test_min_gru_over_portions(N, sched):
    torch.manual_seed(6)
    T = 31
    z, x, g = torch.randn(T, N) * 2, torch.randn(T, N) * 2, torch.randn(T, N)
    a = O.sigmoid(z.double())
    c = torch.where(x.double() >= 0, x.double() + 0.5, O.sigmoid(x.double()))
    S, rows = torch.zeros(N, dtype=F64), []
    for t in range(T):
        S = (1 - a[t]) * S + a[t] * c[t]
        rows.append(S * g[t].double() * O.sigmoid(g[t].double()))
    want = torch.stack(rows)
    state = torch.full((3, N), float("nan"))
    got, at = [], 0
    for n in sched:
        out = torch.zeros(n, N)
        ref.min_gru(z[at:at + n], x[at:at + n], g[at:at + n], state, i32([1]),
                    i32([0, n]), i32(list(range(at, at + n))), out)
        got.append(out)
        at += n
    assert torch.allclose(torch.cat(got).double(), want, atol=1e-5)
    assert torch.allclose(state[1].double(), S, atol=1e-5)


def test_min_gru_candidate_branches_and_far_memory():
    """the candidate is u + 1/2 for u >= 0 and sigmoid(u) below (both meet
    at 1/2); with gates shut after the first token the state is carried
    unchanged over hundreds of tokens"""
    N, T = 2, 300
    z = torch.full((T, N), -60.0)
    z[0] = 60.0
    x = torch.zeros(T, N)
    x[0] = torch.tensor([1.25, -1.25])
    g = torch.full((T, N), 50.0)
    state = torch.zeros(1, N)
    out = torch.zeros(T, N)
    ref.min_gru(z, x, g, state, i32([0]), i32([0, T]), i32(list(range(T))), out)
    want = torch.tensor([1.75, 1 / (1 + math.exp(1.25))])
    assert torch.allclose(out[-1] / 50.0, want, atol=1e-5)
    assert torch.allclose(state[0], want, atol=1e-6)


def test_pair_norm_mean_and_slice_norm():
    torch.manual_seed(7)
    a, b = torch.randn(5, 12) * 4, torch.randn(5, 12) * 0.1
    wa, wb = torch.randn(12), torch.randn(12)
    want = 0.5 * (O.unit(a.double(), 1e-5) * wa.double()
                  + O.unit(b.double(), 1e-5) * wb.double())
    got = ref.pair_rmsnorm_mean(a, wa, b, wb, 1e-5, F32)
    assert torch.allclose(got.double(), want, atol=1e-5)
    # each branch is normed on its own: scaling one leaves its share as is
    got2 = ref.pair_rmsnorm_mean(a * 100, wa, b, wb, 1e-5, F32)
    assert torch.allclose(got2, got, atol=1e-4)
    wide = torch.randn(5, 30)
    sl = wide[:, 7:19]
    assert torch.allclose(ref.slice_rmsnorm(sl, wa, 1e-5).double(),
                          O.unit(sl.double(), 1e-5) * wa.double(), atol=1e-5)


@pytest.mark.parametrize("E,top,n_groups,keep", [(8, 3, 4, 3), (8, 2, 2, 1),
                                                 (6, 1, 3, 2), (4, 4, 1, 1),
                                                 (9, 2, 9, 4), (12, 3, 3, 3)])
def test_routing_matches_oracle(E, top, n_groups, keep):
    torch.manual_seed(8)
    r = {"experts": E, "top": top, "groups": {"count": n_groups, "keep": keep}}
    logits = torch.randn(40, E) * 2
    w, idx = ref.group_topk_gate(logits, top, n_groups, keep, "sigmoid",
                                 min(2, E // n_groups))
    for t in range(40):
        chosen, wts = O.route(logits[t].double(), r)
        assert sorted(chosen) == sorted(idx[t].tolist())
        got = dict(zip(idx[t].tolist(), w[t].tolist()))
        for e, x in zip(chosen, wts):
            assert abs(got[e] - float(x)) < 1e-6


def test_routing_group_score_is_the_sum_of_the_two_best():
    """group 0 holds the single best expert, group 1 the best PAIR: with
    one group kept, the pair's group wins and the best expert is left out;
    the weights are the raw sigmoid scores"""
    logits = torch.tensor([[3.0, -4.0, -4.0, 2.0, 2.0, -4.0]])
    w, idx = ref.group_topk_gate(logits, 2, 2, 1, "sigmoid", 2)
    assert sorted(idx[0].tolist()) == [3, 4]
    assert torch.allclose(w, torch.sigmoid(torch.tensor([[2.0, 2.0]])))
    # with the best single score as the group score, group 0 would win
    _, idx1 = ref.group_topk_gate(logits, 2, 2, 1, "sigmoid", 1)
    assert 0 in idx1[0].tolist()


def test_exact_gelu():
    x = torch.linspace(-6, 6, 101)
    want = O.gelu_erf(x.double())
    assert torch.allclose(ref.gelu_erf(x).double(), want, atol=1e-6)
    # the tanh form differs visibly
    tanh_form = 0.5 * x * (1 + torch.tanh(math.sqrt(2 / math.pi)
                                          * (x + 0.044715 * x ** 3)))
    assert float((tanh_form.double() - want).abs().max()) > 1e-4


def test_config_parsing():
    cfg = O.make_config(kinds=("attention", "parallel", "latent_attention",
                               "parallel"), loop=(1, 3, 3), no_mlp=(2,))
    spec = zevilorn_spec("z", cfg)
    runs = spec.layer_specs
    assert [l.src for l in runs] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [l.weights_of for l in runs] == [None, None, None, 1, 2, 1, 2, None]
    assert [l.readd_embed for l in runs] == [False, False, False, True, False,
                                             True, False, False]
    a = runs[0].mixer
    assert (a.kind, a.score_mix, a.zero_sink, a.bias, a.taps, a.head_gate) == \
        ("gqa_attention", True, True, True, 3, False)
    assert a.rope_scaling["kind"] == "banded" and a.softcap == 2.5
    p = runs[1].mixer
    assert p.combine == "normed_mean" and p.right.width == 13
    assert (p.left.head_gate, p.left.score_mix, p.left.zero_sink, p.left.bias,
            p.left.taps) == (True, False, False, False, 0)
    assert p.left.rope_scaling == {"kind": "linear", "factor": 2.0}
    la = runs[2].mixer
    assert (la.window, la.sink, la.q_rank) == (0, True, 9)
    assert runs[2].ffn is None and runs[0].ffn.group_top == 2
    assert runs[0].ffn.act == "gelu" and runs[0].ffn.score == "sigmoid_all"
    # absent keys: no loop, no rotation, no window, no cap, no conv
    cfg2 = O.make_config(kinds=("attention",), loop=None, rot_dims=0,
                         softcap=0, conv=0)
    del cfg2["layers"][0]["mixer"]["mask"]
    m = zevilorn_spec("z", cfg2).layer_specs[0].mixer
    assert (m.window, m.rope_dims, m.softcap, m.taps) == (0, 0, 0.0, 0)
    for bad in ({"loop": {"start": 2, "stop": 1, "times": 2}},):
        with pytest.raises(ValueError):
            zevilorn_spec("z", dict(cfg, **bad))
    cfg3 = O.make_config(experts=8, n_groups=3)
    with pytest.raises(ValueError):
        zevilorn_spec("z", cfg3)
    cfg4 = O.make_config(kinds=("retention",), loop=None)
    with pytest.raises(ValueError):
        zevilorn_spec("z", cfg4)


# ------------------------------------------------------------ the model

VARIANTS = {
    "base": dict(),
    # values that other models make equal or 1
    "ones": dict(heads=1, kv_heads=1, dim=2, vdim=2, window=1, rot_dims=2,
                 conv=1, lat_heads=1, lat_dim=1, rot_dim=2, lat_vdim=1,
                 kv_rank=1, q_rank=1, left_heads=1, left_kv=1, left_dim=2,
                 left_vdim=1, left_window=1, left_rot=2, gru=1, experts=2,
                 top=1, n_groups=2, keep=1, ff=1, loop=(0, 1, 1)),
    "equal": dict(width=16, heads=4, kv_heads=4, dim=8, vdim=8, window=16,
                  rot_dims=8, lat_heads=4, lat_dim=8, rot_dim=8, lat_vdim=8,
                  kv_rank=8, q_rank=8, left_heads=4, left_kv=4, left_dim=8,
                  left_vdim=8, left_window=16, left_rot=8, gru=16, experts=4,
                  top=4, n_groups=1, keep=1, ff=16, loop=(0, 3, 2)),
    "no-loop": dict(kinds=("parallel", "attention", "latent_attention",
                           "attention"), loop=None, heads=6, kv_heads=1,
                    dim=4, vdim=12, window=33, rot_dims=2, scaling=False,
                    conv=5, softcap=0, no_mlp=(1,), experts=9, top=2,
                    n_groups=3, keep=1, left_rot=0, left_window=40),
    "loop-at-end": dict(kinds=("latent_attention", "parallel", "attention"),
                        loop=(2, 3, 3), conv=2, window=5, left_window=3,
                        experts=6, top=3, n_groups=6, keep=4, heads=8,
                        kv_heads=4, left_heads=6, left_kv=3, no_mlp=(0,)),
}


def _cfg(name):
    return O.make_config(**VARIANTS[name])


@pytest.mark.parametrize("name", list(VARIANTS))
def test_served_model_matches_oracle(tmp_path, name):
    cfg = _cfg(name)
    W = O.random_weights(cfg, seed=11)
    eng = make_engine(tmp_path, cfg, W)
    toks = random_tokens(45, cfg["vocab"], 1)
    want = oracle_logits(cfg, W, toks)
    schedules = {
        "whole": [[("a", 45)]],
        "decode": [[("a", 9)]] + [[("a", 1)]] * 36,
        "portions": chunk_schedule("a", 45, [2, 5, 1, 16, 3]),
        "twos": chunk_schedule("a", 45, [2]),
        "token-by-token": [[("a", 1)]] * 45,
    }
    for what, sched in schedules.items():
        got = replay(eng, {"a": toks}, sched)["a"]
        assert_logits(got, want, F32, what)
    assert eng.kv.free_blocks == eng.kv.n_blocks - 1     # scratch page only


def test_layer_residuals_match_oracle(tmp_path):
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=12)
    eng = make_engine(tmp_path, cfg, W)
    toks = random_tokens(19, cfg["vocab"], 2)
    layers = []
    O.forward(cfg, W, toks, layers)
    seen = []
    eng.runner.layer_tap = lambda i, x: seen.append(x.clone())
    got = eng.feed([("a", toks, list(range(19)))], ["a"])
    assert len(seen) == len(layers) == 5          # 1 + 2 x 2 runs
    for i, x in enumerate(seen):
        assert torch.allclose(x.double(), layers[i], atol=1e-3), i
    # the probe's unfused path and the fused path give the same logits
    eng.runner.layer_tap = None
    again = eng.feed([("b", toks, list(range(19)))], ["b"])
    assert rel_err(again, got) < 1e-5


def test_passes_share_tensors_not_pages_or_state(tmp_path):
    """A repeated block runs the same tensors with pages and state of its
    own per pass; the embedding output is added before the later passes."""
    cfg = _cfg("base")                    # layers 1-2 run twice
    W = O.random_weights(cfg, seed=19)
    eng = make_engine(tmp_path, cfg, W)
    assert eng.weights.layers[3] is eng.weights.layers[1]
    assert eng.weights.layers[4] is eng.weights.layers[2]
    assert eng.kv.k_cache[3] is not eng.kv.k_cache[1]
    assert eng.kv.rec_state[4] is not eng.kv.rec_state[2]
    toks = random_tokens(30, cfg["vocab"], 7)
    want = oracle_logits(cfg, W, toks)
    got = replay(eng, {"a": toks}, [[("a", 4)]] + [[("a", 1)]] * 26)["a"]
    assert_logits(got, want, F32)
    # without the add before the second pass the logits differ
    once = dict(cfg, loop={"start": 1, "stop": 3, "times": 1})
    assert rel_err(oracle_logits(once, W, toks), want) > 1e-3


def test_mixed_batches_and_reuse(tmp_path):
    """Unequal requests side by side (portions next to single tokens, a
    request sitting out a step) equal each request alone; the pool is far
    smaller than the sum of the requests, so pages and slots come back."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=13)
    eng = make_engine(tmp_path, cfg, W, kv_blocks=7, block_size=8,
                      max_batch=3)
    # reused pages and slots hold garbage, never zeros
    for t in eng.kv.k_cache + eng.kv.v_cache + eng.kv.rec_state + \
            eng.kv.conv_state:
        if t is not None:
            t.fill_(float("nan"))
    lens = [21, 6, 30, 11, 17, 2, 26]
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 20 + i)
            for i, n in enumerate(lens)}
    sched = [
        [("r0", 9), ("r1", 2)],
        [("r0", 1), ("r1", 3), ("r2", 5)],
        [("r0", 11), ("r2", 1)],                    # r1 sits out; r0 ends
        [("r1", 1), ("r2", 2), ("r3", 11)],         # r1, r3 end
        [("r2", 22), ("r4", 2)],                    # r2 ends
        [("r4", 15), ("r5", 2), ("r6", 3)],         # r4, r5 end
        [("r6", 1)], [("r6", 22)],
    ]
    got = replay(eng, reqs, sched)
    for rid, toks in reqs.items():
        assert_logits(got[rid], oracle_logits(cfg, W, toks), F32, rid)
    assert eng.kv.free_blocks == eng.kv.n_blocks - 1
    assert eng.kv.free_state_slots == eng.kv.n_state_slots - 1


def test_long_decode_crosses_pages_and_windows(tmp_path):
    cfg = _cfg("base")                    # windows 9 and 7, pages of 4
    W = O.random_weights(cfg, seed=14)
    eng = make_engine(tmp_path, cfg, W, block_size=4, kv_blocks=50)
    toks = random_tokens(140, cfg["vocab"], 3)
    got = replay(eng, {"a": toks}, [[("a", 3)]] + [[("a", 1)]] * 137)["a"]
    assert_logits(got, oracle_logits(cfg, W, toks), F32)


def test_first_tokens_after_page_and_slot_reuse(tmp_path):
    """A request that takes over the pages and the slot another one just
    left must not see anything of it in its first tokens (conv rows,
    recurrent state, keys)."""
    cfg = _cfg("no-loop")
    W = O.random_weights(cfg, seed=15)
    eng = make_engine(tmp_path, cfg, W, max_batch=1, kv_blocks=3, block_size=16)
    a, b = random_tokens(40, cfg["vocab"], 4), random_tokens(6, cfg["vocab"], 5)
    replay(eng, {"a": a}, [[("a", 40)]])
    for sched in ([[("b", 6)]], [[("b", 1)]] * 6, [[("b", 2)], [("b", 4)]]):
        got = replay(eng, {"b": b}, sched)["b"]
        assert_logits(got, oracle_logits(cfg, W, b), F32)


def test_greedy_generation_through_scheduler(tmp_path):
    """submit()/generate(): admission, chunked prompt prefill (budget of 7
    tokens a step), batched decode of concurrent requests, retirement."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=16)
    eng = make_engine(tmp_path, cfg, W, max_prefill_tokens=7)
    try:
        from bee2bee_amd.engine.engine import GenerationRequest
        from bee2bee_amd.engine.sampler import SamplingParams

        prompts = [random_tokens(n, cfg["vocab"], 30 + n) for n in (17, 3, 9)]
        reqs = [eng.submit(GenerationRequest(
            prompt_ids=list(p), max_new_tokens=10,
            sampling=SamplingParams(greedy=True))) for p in prompts]
        for r in reqs:
            while r.done_ts is None:
                r.out_queue.get(timeout=60)
        for p, r in zip(prompts, reqs):
            assert len(r.output_ids) == 10 and r.error is None
            seq = list(p)
            for tok in r.output_ids:
                logits = oracle_logits(cfg, W, seq)[-1]
                top2 = torch.topk(logits, 2).values
                if float(top2[0] - top2[1]) > 1e-3:
                    assert int(logits.argmax()) == tok
                seq.append(tok)
    finally:
        eng.shutdown()


def test_trace_replay_writes_wanted_logits(tmp_path, monkeypatch, capsys):
    from bee2bee_amd.engine import trace

    cfg = _cfg("loop-at-end")
    W = O.random_weights(cfg, seed=17)
    O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    toks = random_tokens(12, cfg["vocab"], 6)
    steps = [
        {"step": 0, "entries": [{"id": "q", "tokens": toks[:7], "want": [0, 6]}],
         "end": []},
        {"step": 1, "entries": [{"id": "q", "tokens": toks[7:8], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "q", "tokens": toks[8:], "want": [3]}],
         "end": ["q"]},
    ]
    monkeypatch.setattr(sys, "stdin", io.StringIO(
        "\n".join(json.dumps(s) for s in steps) + "\n"))
    out = tmp_path / "out"
    assert trace.main(["--model", str(tmp_path / "m"), "--dtype", "float32",
                       "--out", str(out), "--max-tokens", "64"]) == 0
    assert capsys.readouterr().out.split() == ["done", "0", "done", "1",
                                               "done", "2"]
    import numpy as np

    want = oracle_logits(cfg, W, toks)
    a = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
    c = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (out / "1.f32").exists()
    assert rel_err(a, want[[0, 6]]) < 2e-4 and rel_err(c, want[[11]]) < 2e-4


def test_checkpoint_roundtrip(tmp_path):
    """load -> save_hf -> load: the same tensors under the same names, the
    same config, the same layer runs."""
    from safetensors.torch import load_file

    from bee2bee_amd.models.weights import save_hf

    for name in ("base", "no-loop"):
        cfg = _cfg(name)
        W = O.random_weights(cfg, seed=18)
        eng = make_engine(tmp_path / name, cfg, W)
        out = tmp_path / name / "resaved"
        save_hf(eng.weights, str(out))
        W2 = load_file(str(out / "model.safetensors"))
        assert set(W2) == set(W)
        for k in W2:
            assert torch.equal(W2[k].float(), W[k].float()), k
        cfg2 = json.load(open(out / "config.json"))
        a, b = zevilorn_spec("a", cfg), zevilorn_spec("b", cfg2)
        assert a.layer_specs == b.layer_specs
        assert (a.vocab_size, a.hidden_size, a.rms_eps) == \
            (b.vocab_size, b.hidden_size, b.rms_eps)


def test_random_init_runs_and_is_consistent():
    """Synthetic serving (no checkpoint): random weights of a synthetic
    stack; decoding token by token equals the whole prompt."""
    from bee2bee_amd.engine.engine import InferenceEngine
    from bee2bee_amd.models.hybrid import zevilorn_layer_cfgs

    layers = zevilorn_layer_cfgs(3, 32, heads=4, kv_heads=2, dim=8, window=12,
                                 kv_rank=12, rot_dim=4, q_rank=10,
                                 gru_width=20, experts=4, top_k=2,
                                 expert_ff=16, groups=2, keep=1, taps=3)
    spec = zevilorn_spec("zv-synth", {
        "vocab": 64, "width": 32, "norm": {"eps": 1e-6}, "layers": layers,
        "loop": {"start": 1, "stop": 3, "times": 2}, "max_seq_len": 256})
    eng = InferenceEngine(spec, device="cpu", dtype=F32, max_batch=2,
                          max_seq_len=256, use_graphs=False, kv_block_size=8,
                          kv_blocks=16, kv_margin_blocks=1)
    toks = random_tokens(20, 64, 9)
    whole = replay(eng, {"a": toks}, [[("a", 20)]])["a"]
    steps = replay(eng, {"a": toks}, [[("a", 1)]] * 20)["a"]
    assert rel_err(steps, whole) < 1e-4
    assert spec.n_params() > 0
    # the repeated block's tensors count once, its runs every time
    assert spec.active_params_per_token() > 0


def test_bench_compare_option_runs_on_cpu():
    """bench.py --compare-zevilorn: one JSON line per model with prefill
    and decode throughput (CPU run: small stand-in sizes)."""
    import os
    import subprocess

    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(
        [sys.executable, os.path.join(repo, "bench.py"), "--compare-zevilorn",
         "s", "--steps", "1", "--warmup", "0"],
        capture_output=True, text=True, timeout=300,
        env=dict(os.environ, HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES=""))
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(x) for x in r.stdout.splitlines() if x.startswith("{")]
    assert [x["model"] for x in lines] == ["zevilorn-s", "gqa-moe-s"]
    for x in lines:
        assert x["compare"] == "zevilorn-vs-dense"
        assert x["prefill_tokens_per_s"] > 0 and x["decode_tokens_per_s"] > 0
