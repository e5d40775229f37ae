"""Zevilorn served on the GPU (HIP kernels, bf16 and fp32) against the plain
whole-sequence oracle: whole prompts, portions, decode, mixed batches with
page and slot reuse, greedy generation through the scheduler, captured
decode, long portions (the minGRU's segment form, the attention key
splits) and the matrix-core attention paths at their head sizes."""
import pytest
import torch

from tests import zevilorn_oracle as O
from tests.zevilorn_util import (assert_logits, chunk_schedule, make_engine,
                                 oracle_logits, random_tokens, replay)

pytestmark = pytest.mark.gpu

if not torch.cuda.is_available():
    pytest.skip("needs a GPU", allow_module_level=True)

from tests.test_zevilorn import VARIANTS, _cfg  # noqa: E402


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_chunked_decode_match_oracle(tmp_path, dtype):
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=1)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=dtype)
    toks = random_tokens(61, cfg["vocab"], 5)
    want = oracle_logits(cfg, W, toks)
    for sched in ([[("a", 61)]],
                  chunk_schedule("a", 61, [2, 17, 3, 1, 1, 16]),
                  [[("a", 20)]] + [[("a", 1)]] * 41):
        got = replay(eng, {"a": toks}, sched)["a"]
        assert_logits(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_batches_reuse_pages_and_slots(tmp_path, dtype):
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=2)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=dtype,
                      kv_blocks=12, block_size=16)
    for t in eng.kv.k_cache + eng.kv.v_cache + eng.kv.rec_state + \
            eng.kv.conv_state:
        if t is not None:
            t.fill_(float("nan"))
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 10 + i)
            for i, n in enumerate([37, 9, 52, 18, 33, 5, 41])}
    sched = [
        [("r0", 20), ("r1", 2)],
        [("r0", 1), ("r1", 7), ("r2", 30)],
        [("r0", 16), ("r2", 1), ("r3", 18)],        # r0, r1, r3 end
        [("r2", 21), ("r4", 33), ("r5", 2), ("r6", 3)],
        [("r5", 3), ("r6", 38)],
    ]
    got = replay(eng, reqs, sched)
    for rid, toks in reqs.items():
        assert_logits(got[rid], oracle_logits(cfg, W, toks), dtype, rid)
    assert eng.kv.free_blocks == eng.kv.n_blocks - 1
    assert eng.kv.free_state_slots == eng.kv.n_state_slots - 1


@pytest.mark.parametrize("name", list(VARIANTS))
def test_variants_fp32(tmp_path, name):
    cfg = _cfg(name)
    W = O.random_weights(cfg, seed=21)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=torch.float32)
    toks = random_tokens(45, cfg["vocab"], 1)
    want = oracle_logits(cfg, W, toks)
    for sched in ([[("a", 45)]], chunk_schedule("a", 45, [2, 5, 1, 16, 3]),
                  [[("a", 9)]] + [[("a", 1)]] * 36):
        assert_logits(replay(eng, {"a": toks}, sched)["a"], want,
                      torch.float32, name)


def test_long_portions_and_key_splits(tmp_path):
    """A portion long enough for the minGRU's segment form and decode rows
    over a context long enough for the attention key splits, without
    windows, fp32 against the oracle."""
    cfg = O.make_config(window=0, left_window=0, loop=(0, 3, 2))
    for l in cfg["layers"]:
        m = l["mixer"].get("left", l["mixer"])
        m.pop("mask", None)
    W = O.random_weights(cfg, seed=24)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=torch.float32,
                      kv_blocks=40)
    toks = random_tokens(330, cfg["vocab"], 9)
    want = oracle_logits(cfg, W, toks)
    for sched in ([[("a", 300)]] + [[("a", 1)]] * 30,
                  [[("a", 150)], [("a", 170)]] + [[("a", 1)]] * 10):
        got = replay(eng, {"a": toks}, sched)["a"]
        assert_logits(got, want, torch.float32)


def test_greedy_generation_through_scheduler(tmp_path):
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=3)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=torch.float32)
    try:
        prompt = random_tokens(11, cfg["vocab"], 3)
        req = eng.generate(prompt, max_new_tokens=12, temperature=0.0,
                           repetition_penalty=1.0)
        seq = list(prompt)
        for tok in req.output_ids:
            logits = oracle_logits(cfg, W, seq)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > 1e-3:   # skip near-ties
                assert int(logits.argmax()) == tok
            seq.append(tok)
        assert len(req.output_ids) == 12
    finally:
        eng.shutdown()


def test_graph_decode_equals_eager(tmp_path):
    """Captured decode steps (hipGraph) replayed several times with eager
    prefill work between them must give the tokens of the eager engine."""
    cfg = _cfg("base")
    W = O.random_weights(cfg, seed=23)
    prompts = [random_tokens(n, cfg["vocab"], 40 + n) for n in (13, 5)]
    outs = {}
    for graphs in (False, True):
        eng = make_engine(tmp_path, cfg, W, device="cuda",
                          dtype=torch.float32, use_graphs=graphs)
        assert (eng.graphs is not None) == graphs
        try:
            outs[graphs] = [
                eng.generate(p, max_new_tokens=24, temperature=0.0,
                             repetition_penalty=1.0).output_ids
                for p in prompts]
        finally:
            eng.shutdown()
    assert outs[True] == outs[False]
    seq = list(prompts[0])
    for tok in outs[True][0]:
        logits = oracle_logits(cfg, W, seq)[-1]
        top2 = torch.topk(logits, 2).values
        if float(top2[0] - top2[1]) > 1e-3:
            assert int(logits.argmax()) == tok
        seq.append(tok)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("left_kv,left_window", [(2, 50), (4, 0)])
def test_head_sizes_of_the_matrix_core_paths(tmp_path, dtype, left_kv,
                                             left_window):
    """Heads of 64 in both grouped-query attentions (score-mixing and
    windowed) and a latent row of 64 + 32:
    bf16 prompt portions of 16 tokens or more run on the matrix cores,
    shorter portions and decode rows on the generic kernels with their key
    splits; fp32 takes the generic kernels throughout. All must agree with
    the oracle on one sequence cut in different ways."""
    cfg = O.make_config(width=64, vocab=90, ff=24, heads=4, kv_heads=2,
                        dim=64, vdim=64, rot_dims=32, window=70,
                        lat_heads=4, lat_dim=16, rot_dim=32, lat_vdim=16,
                        kv_rank=64, q_rank=24, left_heads=4, left_kv=left_kv,
                        left_dim=64, left_vdim=64, left_window=left_window,
                        left_rot=32, gru=40, loop=(1, 3, 2))
    if not left_window:
        cfg["layers"][2]["mixer"]["left"].pop("mask")
    W = O.random_weights(cfg, seed=25)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=dtype,
                      kv_blocks=40)
    toks = random_tokens(210, cfg["vocab"], 11)
    want = oracle_logits(cfg, W, toks)
    for sched in ([[("a", 210)]],
                  chunk_schedule("a", 210, [100, 3, 60, 17, 1, 16]),
                  [[("a", 170)]] + [[("a", 1)]] * 40):
        got = replay(eng, {"a": toks}, sched)["a"]
        assert_logits(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_expert_execution_strategies(tmp_path, dtype):
    """Steps of 300 and 700 tokens at a width and expert size the
    grouped-GEMM kernel covers (bf16: sorted token slots through the kernel;
    beyond its range and in fp32 the per-expert loop), decode rows through
    the dense all-experts product: all equal the oracle."""
    cfg = O.make_config(width=128, vocab=80, ff=128, experts=8, top=2,
                        n_groups=4, keep=2, kinds=("parallel", "attention"),
                        loop=None, gru=24)
    W = O.random_weights(cfg, seed=26)
    eng = make_engine(tmp_path, cfg, W, device="cuda", dtype=dtype,
                      kv_blocks=80)
    toks = random_tokens(1010, cfg["vocab"], 12)
    want = oracle_logits(cfg, W, toks)
    got = replay(eng, {"a": toks},
                 [[("a", 300)], [("a", 700)]] + [[("a", 1)]] * 10)["a"]
    assert_logits(got, want, dtype)
