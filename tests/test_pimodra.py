"""Pimodra on the CPU reference path against the plain oracle
(tests/pimodra_oracle.py): each mechanism alone, then the served model —
whole prompts, decoding, portions, mixed batches with page and slot reuse,
window and page edges, the scheduler's own greedy generation."""
import io
import json
import math
import sys

import pytest
import torch

from bee2bee_amd.models.spec import pimodra_spec
from bee2bee_amd.ops import reference as ref
from tests import pimodra_oracle as O
from tests.pimodra_util import (assert_logits, chunk_schedule, make_engine,
                                oracle_logits, random_tokens, rel_err, replay)

F32, F64 = torch.float32, torch.float64


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


# ----------------------------------------------------------- mechanisms

@pytest.mark.parametrize("W,groups", [(12, 1), (12, 3), (30, 5), (8, 8)])
def test_group_norm_and_fused_update(W, groups):
    torch.manual_seed(0)
    x = torch.randn(5, W) * 3
    y = torch.randn(5, W) * 2
    w1, w2, step = torch.randn(W), torch.randn(W), torch.randn(W)
    want_x = x.double() + O.group_norm(y.double(), w1.double(), groups, 1e-5)
    want_x = want_x + step.double()
    want = O.group_norm(want_x, w2.double(), groups, 1e-5)
    r = x.clone()
    got = ref.add_group_rmsnorm(r, y, w1, step, w2, groups, 1e-5, F32)
    assert torch.allclose(r.double(), want_x, atol=1e-5)
    assert torch.allclose(got.double(), want, atol=1e-5)
    # the parts of a row are normed on their own: scaling one part leaves
    # the others' outputs alone
    if groups > 1:
        gw = W // groups
        x2 = x.clone()
        x2[:, :gw] *= 50.0
        a = ref.group_rmsnorm(x, w2, groups, 1e-5, F32)
        b = ref.group_rmsnorm(x2, w2, groups, 1e-5, F32)
        assert torch.allclose(a[:, gw:], b[:, gw:], atol=1e-6)
    # step only, norm only, nothing to return
    r2 = x.clone()
    assert ref.add_group_rmsnorm(r2, None, None, step, None, groups, 1e-5,
                                 F32) is None
    assert torch.allclose(r2, x + step)


@pytest.mark.parametrize("scaling", [
    None, {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 0.5},
    {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0},
    {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}])
@pytest.mark.parametrize("dims,base", [(4, 500.0), (16, 10000.0), (2, 7.0)])
def test_rotation_tables(scaling, dims, base):
    rot = {"dims": dims, "base": base}
    if scaling:
        rot["scaling"] = scaling
    freq, mag = O.rope_frequencies(rot)
    cos, sin = ref.rope_tables_scaled(40, dims, base, scaling, "cpu")
    for p in (0, 1, 17, 39):
        for i in range(dims // 2):
            assert abs(float(cos[p, i]) - math.cos(p * freq[i]) * mag) < 1e-6
            assert abs(float(sin[p, i]) - math.sin(p * freq[i]) * mag) < 1e-6


def _paged(seq_len, bs, n_blocks, seed):
    g = torch.Generator().manual_seed(seed)
    need = -(-seq_len // bs)
    return torch.randperm(n_blocks, generator=g)[:need].to(torch.int32)


def _attend(q, k, v, talk, gate, rot, eps, scale, window, cuts, bs=8):
    """Run [q k v] of one sequence through rope_unit_store + talk_attn in
    portions `cuts` over scattered pages; returns [T, H*Dv]."""
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    nb = -(-T // bs) + 3
    table = _paged(T, bs, nb, 1)
    kc = torch.full((nb, G, bs, D), float("nan"))
    vc = torch.full((nb, G, bs, Dv), float("nan"))
    dims = rot["dims"] if rot else 0
    cos = sin = None
    if rot:
        cos, sin = ref.rope_tables_scaled(T + 1, dims, rot["base"],
                                          rot.get("scaling"), "cpu")
    out = torch.zeros(T, H * Dv)
    at = 0
    for n in cuts:
        pos = i32(list(range(at, at + n)))
        slots = i32([int(table[p // bs]) * bs + p % bs
                     for p in range(at, at + n)])
        qq = q[at:at + n].clone()
        ref.rope_unit_store(qq, k[at:at + n], v[at:at + n], eps, dims, pos,
                            cos, sin, scale, kc, vc, slots)
        o = torch.zeros(n, H * Dv)
        ref.talk_attn(qq, kc, vc, table[None], pos, i32([0] * n), i32([0, n]),
                      talk, gate[at:at + n], window, o)
        out[at:at + n] = o
        at += n
    return out


def _oracle_attend(q, k, v, talk, gate, rot, eps, scale, window):
    T, H, _ = q.shape
    G, Dv = k.shape[1], v.shape[2]
    qd, kd = q.double(), k.double()
    if rot:
        qd, kd = O.rotate(qd, rot), O.rotate(kd, rot)
    w = O.attention_weights(O.unit(qd, eps), O.unit(kd, eps), scale,
                            window or None)
    w = torch.einsum("hg,gij->hij", talk.double(), w)
    o = torch.stack([w[h] @ v[:, h // (H // G)].double() for h in range(H)], 1)
    return o.reshape(T, H * Dv) * torch.sigmoid(gate.double())


@pytest.mark.parametrize("cuts", [[50], [2, 7, 1, 24, 16], [1] * 50])
@pytest.mark.parametrize("H,G,D,Dv,dims,window", [
    (4, 2, 6, 10, 4, 9), (3, 3, 8, 8, 8, 0), (6, 1, 4, 3, 0, 17),
    (2, 2, 10, 4, 2, 1)])
def test_talk_attention_matches_oracle(cuts, H, G, D, Dv, dims, window):
    torch.manual_seed(3)
    T = 50
    q, k = torch.randn(T, H, D), torch.randn(T, G, D)
    v = torch.randn(T, G, Dv)
    talk = torch.eye(H) + 0.4 * torch.randn(H, H)
    gate = torch.randn(T, H * Dv)
    rot = {"dims": dims, "base": 300.0,
           "scaling": {"factor": 4.0, "original": 12, "fast": 3.0,
                       "slow": 0.5}} if dims else None
    got = _attend(q, k, v, talk, gate, rot, 1e-6, 0.8, window, cuts)
    want = _oracle_attend(q, k, v, talk, gate, rot, 1e-6, 0.8, window)
    assert torch.allclose(got.double(), want, atol=2e-5)


def test_head_mixing_uses_own_values_and_all_weights():
    """Head h's output is its OWN value head read with a mixture of every
    head's weights: with talk = one-hot rows pointing at another head, head
    h reproduces that head's attention pattern on h's values."""
    torch.manual_seed(4)
    T, H, G, D, Dv = 12, 4, 2, 6, 5
    q, k, v = torch.randn(T, H, D), torch.randn(T, G, D), torch.randn(T, G, Dv)
    gate = torch.full((T, H * Dv), 30.0)          # gate ~ 1
    perm = [3, 2, 1, 0]                           # head h takes head perm[h]
    talk = torch.zeros(H, H)
    for h, g in enumerate(perm):
        talk[h, g] = 1.0
    got = _attend(q, k, v, talk, gate, None, 1e-6, 1.0, 0, [T]).view(T, H, Dv)
    w = O.attention_weights(O.unit(q.double(), 1e-6), O.unit(k.double(), 1e-6),
                            1.0, None)
    for h in range(H):
        want = w[perm[h]] @ v[:, h // 2].double()
        assert torch.allclose(got[:, h].double(), want, atol=1e-5), h
    # the gate multiplies element by element, after the mix
    gate2 = torch.zeros(T, H * Dv)
    half = _attend(q, k, v, talk, gate2, None, 1e-6, 1.0, 0, [T])
    assert torch.allclose(half, 0.5 * got.reshape(T, -1), atol=1e-5)


@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("far", [0, 7, 8, 63, 64, 200])
def test_far_key_among_hundreds(decoded, far):
    """One key far back is made to stand out for the last query: the output
    must be that key's value — first token, both sides of page borders."""
    torch.manual_seed(5)
    T, H, G, D, Dv = 260, 2, 1, 8, 4
    q, k = 0.05 * torch.randn(T, H, D), 0.05 * torch.randn(T, G, D)
    v = torch.randn(T, G, Dv)
    d = torch.zeros(D)
    d[3] = 1.0
    k[:, :, 3] = 0.0                 # no other key points that way
    k[far, 0] = 5 * d
    q[T - 1, :] = 5 * d
    talk = torch.eye(H)
    gate = torch.full((T, H * Dv), 30.0)
    cuts = [T - 40] + [1] * 40 if decoded else [100, 160]
    got = _attend(q, k, v, talk, gate, None, 1e-6, 12.0, 0, cuts, bs=8)
    want = _oracle_attend(q, k, v, talk, gate, None, 1e-6, 12.0, 0)
    assert torch.allclose(got.double(), want, atol=1e-5)
    # unit-norm q.k = D * cos: score 96 against ~0 -> all weight on `far`
    assert torch.allclose(got[T - 1].view(H, Dv)[0], v[far, 0], atol=1e-3)


@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("window", [1, 5, 16, 17])
def test_window_edges(decoded, window):
    """A dominant key just inside the window takes the weight; one position
    further back it is not seen at all."""
    torch.manual_seed(6)
    T, H, G, D, Dv = 60, 2, 2, 8, 3
    for back, seen in ((window - 1, True), (window, False)):
        q, k = 0.05 * torch.randn(T, H, D), 0.05 * torch.randn(T, G, D)
        v = torch.randn(T, G, Dv)
        d = torch.zeros(D)
        d[1] = 1.0
        k[:, :, 1] = 0.0
        j = T - 1 - back
        k[j, :] = 5 * d
        q[T - 1, :] = 5 * d
        v[j] = 100.0
        talk = torch.eye(H)
        gate = torch.full((T, H * Dv), 30.0)
        cuts = [T - 20] + [1] * 20 if decoded else [T]
        got = _attend(q, k, v, talk, gate, None, 1e-6, 12.0, window, cuts)
        want = _oracle_attend(q, k, v, talk, gate, None, 1e-6, 12.0, window)
        assert torch.allclose(got.double(), want, atol=1e-4)
        last = got[T - 1]
        assert bool((last > 99).all()) == seen, (back, last)


def test_polynorm_matches_formula():
    torch.manual_seed(7)
    z = torch.randn(6, 20) * 1.5
    coef = torch.tensor([0.4, -0.3, 0.2, 0.05])
    want = O.polynorm(z.double(), coef.double(), 1e-6)
    assert torch.allclose(ref.polynorm(z, coef, 1e-6, F32).double(), want,
                          atol=1e-5)
    # each power has its own norm: the cube term is scale-free
    c3 = torch.tensor([0.0, 0.0, 1.0, 0.0])
    a = ref.polynorm(z, c3, 0.0, F32)
    b = ref.polynorm(7 * z, c3, 0.0, F32)
    assert torch.allclose(a, b, atol=1e-5)


@pytest.mark.parametrize("E,top,n_g,keep", [(6, 2, 3, 2), (8, 3, 4, 2),
                                            (4, 4, 1, 1), (6, 1, 6, 1),
                                            (9, 3, 3, 3)])
def test_group_limited_routing(E, top, n_g, keep):
    torch.manual_seed(8)
    h = torch.randn(40, 12)
    router = torch.randn(E, 12)
    r = {"experts": E, "top": top, "groups": {"count": n_g, "keep": keep}}
    want = O.route(h.double(), router.double(), r)
    w, idx = ref.group_topk_gate(h @ router.T, top, n_g, keep)
    got = torch.zeros(40, E).scatter_(1, idx.long(), w)
    assert torch.allclose(got.double(), want, atol=1e-6)
    # weights are softmax scores over all experts, not renormalized
    assert float(w.sum(-1).max()) < 1.0 or top == E


def test_best_expert_outside_kept_groups_is_not_chosen():
    # groups {0,1} {2,3} {4,5}; keep 1: group score = its best expert
    z = torch.tensor([[0.0, 3.0, 2.9, 2.9, -1.0, -1.0]])
    w, idx = ref.group_topk_gate(z, 2, 3, 1)
    assert sorted(idx[0].tolist()) == [0, 1]
    s = torch.softmax(z, -1)
    assert torch.allclose(w.sort().values, s[0, [0, 1]].sort().values)


# ---------------------------------------------------------------- config

def test_config_is_read_not_assumed():
    cfg = O.make_config(heads=6, kv_heads=3, dim=8, vdim=4, window=11,
                        rot_dims=6, kinds=("moe", None, "dense"), groups=3,
                        experts=8, top=3, n_groups=4, keep=3, expert_ff=5,
                        ff=14, loop=(0, 2, 3), width=18, vocab=51)
    s = pimodra_spec("x", cfg)
    assert (s.vocab_size, s.hidden_size, s.norm_groups, s.step_rows) == (
        51, 18, 3, 3)
    assert s.tie_embeddings and s.arch == "pimodra"
    runs = s.layer_specs
    assert [l.src for l in runs] == [0, 1, 0, 1, 0, 1, 2]
    assert [l.step_row for l in runs] == [0, None, 1, None, 2, None, None]
    assert [l.weights_of for l in runs] == [None, None, 0, 1, 0, 1, None]
    m = runs[0].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.window, m.rope_dims) == (
        6, 3, 8, 4, 11, 6)
    assert m.rope_scaling["factor"] == 3.0 and m.rope_base == 500.0
    f = runs[0].ffn
    assert (f.n_experts, f.top_k, f.n_groups, f.keep_groups, f.ff, f.act,
            f.score) == (8, 3, 4, 3, 5, "silu_glu", "softmax_all")
    assert runs[1].ffn is None and runs[6].ffn.ff == 14
    # no loop, no window, no rotation, no scaling
    cfg2 = O.make_config(window=0, rot_dims=0, loop=None, kinds=("dense",))
    s2 = pimodra_spec("y", cfg2)
    m2 = s2.layer_specs[0].mixer
    assert (m2.window, m2.rope_dims, m2.rope_scaling, s2.step_rows) == (
        0, 0, None, 0)
    with pytest.raises(ValueError):
        pimodra_spec("z", O.make_config(experts=6, n_groups=4))
    with pytest.raises(ValueError):
        pimodra_spec("z", O.make_config(loop=(2, 1, 2)))


# ------------------------------------------------------------ the model

VARIANTS = {
    "base": dict(),
    # values that other models make equal or 1
    "ones": dict(heads=2, kv_heads=2, dim=8, vdim=8, groups=1, window=1,
                 rot_dims=8, scaling=False, experts=4, top=1, n_groups=1,
                 keep=1, loop=(0, 1, 1), kinds=("moe", "dense")),
    "single-kv": dict(heads=6, kv_heads=1, dim=4, vdim=12, groups=4,
                      window=0, rot_dims=2, experts=8, top=4, n_groups=4,
                      keep=3, loop=(1, 2, 3), kinds=("dense", "moe")),
    "no-loop": dict(heads=3, kv_heads=3, dim=10, vdim=6, groups=3, width=30,
                    window=33, rot_dims=0, loop=None, experts=3, top=3,
                    n_groups=3, keep=3, kinds=("moe", None, "dense", "moe")),
    "loop-at-end": dict(heads=8, kv_heads=4, dim=6, vdim=4, window=20,
                        rot_dims=6, loop=(2, 3, 2), experts=9, top=2,
                        n_groups=3, keep=1, kinds=("dense", "dense", "moe")),
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


def test_passes_share_tensors_not_pages(tmp_path):
    """A repeated block runs the same tensors with pages of its own per
    pass, and each pass adds its own step row first."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=19)
    eng = make_engine(tmp_path, cfg, W)
    assert eng.weights.layers[3] is eng.weights.layers[1]
    assert eng.weights.layers[4] is eng.weights.layers[2]
    assert eng.kv.k_cache[3] is not eng.kv.k_cache[1]
    toks = random_tokens(30, cfg["vocab"], 7)
    want = oracle_logits(cfg, W, toks)
    got = replay(eng, {"a": toks}, [[("a", 4)]] + [[("a", 1)]] * 26)["a"]
    assert_logits(got, want, F32)
    # the step rows matter: another table gives other logits
    W2 = dict(W)
    W2["loop.step"] = W["loop.step"].flip(0).contiguous()
    assert rel_err(oracle_logits(cfg, W2, toks), want) > 1e-3


def test_mixed_batches_and_reuse(tmp_path):
    """Unequal requests side by side (portions next to single tokens, a
    request sitting out a step) equal each request alone; the pool is far
    smaller than the sum of the requests, so pages and slots come back."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=13)
    eng = make_engine(tmp_path, cfg, W, kv_blocks=7, block_size=8,
                      max_batch=3)
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
    cfg = _cfg("base")                    # window 9, pages of 4
    W = O.random_weights(cfg, seed=14)
    eng = make_engine(tmp_path, cfg, W, block_size=4, kv_blocks=50)
    toks = random_tokens(140, cfg["vocab"], 3)
    got = replay(eng, {"a": toks}, [[("a", 3)]] + [[("a", 1)]] * 137)["a"]
    assert_logits(got, oracle_logits(cfg, W, toks), F32)


def test_first_tokens_after_page_reuse(tmp_path):
    """A request that takes over the pages another one just left must not
    see anything of it in its first tokens."""
    cfg = _cfg("single-kv")               # no window: every key is read
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

    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=18)
    eng = make_engine(tmp_path, cfg, W)
    out = tmp_path / "resaved"
    save_hf(eng.weights, str(out))
    W2 = load_file(str(out / "model.safetensors"))
    assert set(W2) == set(W)
    for k in W2:
        assert torch.equal(W2[k].float(), W[k].float()), k
    cfg2 = json.load(open(out / "config.json"))
    a, b = pimodra_spec("a", cfg), pimodra_spec("b", cfg2)
    assert a.layer_specs == b.layer_specs
    assert (a.vocab_size, a.hidden_size, a.norm_groups, a.rms_eps,
            a.step_rows) == (b.vocab_size, b.hidden_size, b.norm_groups,
                             b.rms_eps, b.step_rows)


def test_random_init_runs_and_is_consistent():
    """Synthetic serving (no checkpoint): random weights of a synthetic
    stack; decoding token by token equals the whole prompt."""
    from bee2bee_amd.engine.engine import InferenceEngine
    from bee2bee_amd.models.hybrid import pimodra_layers
    from bee2bee_amd.models.spec import hybrid_spec

    layers = pimodra_layers(3, 32, heads=4, kv_heads=2, dim=8, window=12,
                            ff=40, experts=4, top_k=2, expert_ff=16,
                            groups=2, keep=1, loop=(1, 3, 2))
    spec = hybrid_spec("pm-synth", 64, 32, layers, eps=1e-6, embed_scale=1.0,
                       canon_taps=0, max_seq_len=256, arch="pimodra",
                       norm_type="group_rmsnorm", act_type="polynorm")
    spec.tie_embeddings, spec.norm_groups, spec.step_rows = True, 2, 2
    eng = InferenceEngine(spec, device="cpu", dtype=F32, max_batch=2,
                          max_seq_len=256, use_graphs=False, kv_block_size=8,
                          kv_blocks=16, kv_margin_blocks=1)
    toks = random_tokens(20, 64, 9)
    whole = replay(eng, {"a": toks}, [[("a", 20)]])["a"]
    steps = replay(eng, {"a": toks}, [[("a", 1)]] * 20)["a"]
    assert rel_err(steps, whole) < 1e-4


def test_bench_compare_option_runs_on_cpu():
    """bench.py --compare-pimodra: one JSON line per model with prefill and
    decode throughput (CPU run: small stand-in sizes)."""
    import os
    import subprocess

    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run(
        [sys.executable, os.path.join(repo, "bench.py"), "--compare-pimodra",
         "s", "--steps", "1", "--warmup", "0"],
        capture_output=True, text=True, timeout=300,
        env=dict(os.environ, HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES=""))
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(x) for x in r.stdout.splitlines() if x.startswith("{")]
    assert [x["model"] for x in lines] == ["pimodra-s", "gqa-moe-s"]
    for x in lines:
        assert x["compare"] == "pimodra-vs-dense"
        assert x["prefill_tokens_per_s"] > 0 and x["decode_tokens_per_s"] > 0
