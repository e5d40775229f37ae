"""Helpers of the Zevilorn tests: write a small random checkpoint, serve it
with the engine; replay/compare helpers are shared with the other hybrid
families' tests."""
from __future__ import annotations

from typing import Sequence

import torch

from tests import zevilorn_oracle as O
from tests.nukopel_util import (assert_logits, chunk_schedule,  # noqa: F401
                                random_tokens, rel_err, replay, row_errs)


def make_engine(tmp_path, cfg, W, device="cpu", dtype=torch.float32,
                max_batch=4, block_size=16, kv_blocks=64, max_seq_len=1024,
                **kw):
    from bee2bee_amd.engine.engine import InferenceEngine

    path = str(tmp_path / "ckpt")
    O.save_checkpoint(path, cfg, W)
    return InferenceEngine(
        "zv-test", device=device, dtype=dtype, model_path=path,
        max_batch=max_batch, max_seq_len=max_seq_len,
        use_graphs=kw.pop("use_graphs", False), kv_block_size=block_size,
        kv_blocks=kv_blocks, kv_margin_blocks=1, **kw)


def oracle_logits(cfg, W, tokens: Sequence[int]) -> torch.Tensor:
    return O.forward(cfg, W, list(tokens))
