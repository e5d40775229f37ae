"""Paged KV cache: fixed-size blocks from a per-layer device pool.

Sized for MI355X's 288 GB HBM3E: the pool is allocated once up front (no
allocator churn in the decode loop, a requirement for hipGraph capture) and
blocks are handed to sequences from a free list. Layout
[n_blocks, n_kv_heads, block_size, head_dim] keeps one (key, head) row
contiguous (256 B for hd=128 bf16) — the decode kernel reads it as 64 lanes
x 4 B, a perfectly coalesced wave read.

Hybrid stacks (spec.layer_specs) get a different pool per layer kind from
the SAME page and slot bookkeeping:
  * latent-attention layers: one page pool [n_blocks, block_size,
    kv_rank + rot_dim] — the normed latent and the shared rotated key part
    of each token (k_cache[i]; there is no separate value pool);
  * sink-attention layers (grouped-query softmax attention whose values
    are the raw key projection): the dense page layout, k_cache[i] holding
    normed+rotated keys and v_cache[i] the keys as projected;
  * head-mixing attention layers: the same two pools, k_cache[i] holding
    rotated unit-norm keys, v_cache[i] the value projection; a layer that
    runs several times (a repeated block) has pools per run;
  * linear-attention / retention / delta-rule layers: no pages, a recurrent
    state [n_slots, heads, dim, vdim] fp32 per sequence slot;
  * every layer with a convolution: the last taps-1 conv inputs
    [n_slots, taps-1, channels] per sequence slot (the mixer input for the
    whole-width conv, the q|k|v projection for a delta mixer's short conv);
  * grouped-query attention with a short convolution on its projected
    q|k|v: the two page pools and the last taps-1 projected rows per slot;
  * an element-wise gated recurrence (minGRU): state [n_slots, width] fp32;
  * a parallel mixer (attention + delta rule or minGRU side by side) has
    pages AND state in the same layer.
A sequence owns one state slot from new_seq to free_seq. Slots and pages
are handed out again without clearing: the kernels never read state or
cache rows that precede a sequence's position 0.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..models.spec import ModelSpec

# 256-token pages: one decode-attention chunk (DEC_CHUNK) spans exactly one
# page, so the KV stream is 64 KB-sequential per (head, chunk) — measured
# 5.19 -> 5.42/5.54 TB/s at B768/B1536 vs 32-token pages (round 2).
# Allocation granularity coarsens (one page = 256 tokens per sequence),
# which the 288 GB pool absorbs.
BLOCK_SIZE = 256


class PagedKV:
    def __init__(
        self,
        spec: ModelSpec,
        device: torch.device,
        dtype: torch.dtype,
        n_blocks: int,
        block_size: int = BLOCK_SIZE,
        layer_range: Optional[Tuple[int, int]] = None,
        kv_dtype: str = "native",
        n_state_slots: int = 0,
    ) -> None:
        """kv_dtype: "native" stores the compute dtype; "fp8" stores OCP
        e4m3 bytes (uint8 pool, HALF the KV bytes — the decode kernels read
        fp8 directly; opt-in, reported separately from the bf16 headline)."""
        self.spec = spec
        self.device = device
        self.dtype = dtype
        self.kv_dtype = kv_dtype
        self.block_size = block_size
        self.n_blocks = n_blocks
        lo, hi = layer_range or (0, spec.n_layers)
        self.layer_lo = lo
        store_dtype = torch.uint8 if kv_dtype == "fp8" else dtype
        self.n_state_slots = 0
        self._free_slots: List[int] = []
        self._seq_slot: Dict[int, int] = {}
        if spec.is_hybrid:
            if kv_dtype != "native" or layer_range is not None:
                raise ValueError(
                    "hybrid stacks use the native cache dtype, unsharded")
            self._init_hybrid(n_state_slots)
        else:
            shape = (n_blocks, spec.n_kv_heads, block_size, spec.head_dim)
            self.k_cache = [
                torch.zeros(shape, device=device, dtype=store_dtype)
                for _ in range(lo, hi)
            ]
            self.v_cache = [
                torch.zeros(shape, device=device, dtype=store_dtype)
                for _ in range(lo, hi)
            ]
        self._free: List[int] = list(range(n_blocks - 1, -1, -1))
        self._seq_blocks: Dict[int, List[int]] = {}
        self._seq_len: Dict[int, int] = {}

    def _init_hybrid(self, n_slots: int) -> None:
        spec, dev = self.spec, self.device
        if n_slots <= 0:
            raise ValueError("hybrid stacks need n_state_slots > 0")
        self.n_state_slots = n_slots
        self._free_slots = list(range(n_slots - 1, -1, -1))
        self.k_cache, self.v_cache = [], []
        self.conv_state: List[Optional[torch.Tensor]] = []
        self.rec_state: List[Optional[torch.Tensor]] = []
        from ..models.hybrid import mixer_parts

        taps = spec.canon_taps
        f32 = torch.float32
        for l in spec.layer_specs:
            k = v = rec = conv = None
            for _, m in mixer_parts(l.mixer):
                if m.kind == "latent_attention":
                    k = torch.zeros(self.n_blocks, self.block_size,
                                    m.cache_dim, device=dev, dtype=self.dtype)
                elif m.kind in ("sink_attention", "talk_attention",
                                "gqa_attention"):
                    # the dense models' page layout: one (key, head) row
                    # contiguous; values here are the raw key projection
                    k = torch.zeros(self.n_blocks, m.kv_heads,
                                    self.block_size, m.dim, device=dev,
                                    dtype=self.dtype)
                    v = torch.zeros(self.n_blocks, m.kv_heads,
                                    self.block_size, m.vdim, device=dev,
                                    dtype=self.dtype)
                    if m.kind == "gqa_attention" and m.taps > 1:
                        # the last taps-1 projected q|k|v rows
                        conv = torch.zeros(n_slots, m.taps - 1,
                                           m.conv_channels, device=dev,
                                           dtype=self.dtype)
                elif m.kind == "min_gru":
                    rec = torch.zeros(n_slots, m.width, device=dev,
                                      dtype=f32)
                else:   # lightning / retention / delta: recurrent state
                    rec = torch.zeros(n_slots, m.heads, m.dim, m.vdim,
                                      device=dev, dtype=f32)
                    if m.kind == "delta" and m.taps > 1:
                        conv = torch.zeros(n_slots, m.taps - 1,
                                           m.conv_channels, device=dev,
                                           dtype=self.dtype)
            if l.form == "sandwich" and taps >= 1:
                conv = torch.zeros(n_slots, taps - 1, spec.hidden_size,
                                   device=dev, dtype=self.dtype)
            self.k_cache.append(k)
            self.v_cache.append(v)
            self.rec_state.append(rec)
            self.conv_state.append(conv)

    # ------------------------------------------------------- state slots

    @property
    def free_state_slots(self) -> int:
        return len(self._free_slots)

    def state_slot(self, seq_id: int) -> int:
        return self._seq_slot[seq_id]

    def state_slots(self, seq_ids: Sequence[int]) -> torch.Tensor:
        """[B] int32 device tensor of the sequences' state slots."""
        return torch.tensor([self._seq_slot[s] for s in seq_ids],
                            dtype=torch.int32).to(self.device,
                                                  non_blocking=True)

    def layer(self, layer_idx: int) -> Tuple[torch.Tensor, torch.Tensor]:
        return self.k_cache[layer_idx - self.layer_lo], self.v_cache[layer_idx - self.layer_lo]

    @property
    def free_blocks(self) -> int:
        return len(self._free)

    def new_seq(self, seq_id: int) -> None:
        if seq_id in self._seq_blocks:
            self.free_seq(seq_id)
        if self.n_state_slots:
            if not self._free_slots:
                raise RuntimeError(
                    f"state slots exhausted ({self.n_state_slots})")
            self._seq_slot[seq_id] = self._free_slots.pop()
        self._seq_blocks[seq_id] = []
        self._seq_len[seq_id] = 0

    def free_seq(self, seq_id: int) -> None:
        blocks = self._seq_blocks.pop(seq_id, [])
        self._seq_len.pop(seq_id, None)
        self._free.extend(reversed(blocks))
        slot = self._seq_slot.pop(seq_id, None)
        if slot is not None:
            self._free_slots.append(slot)

    def seq_len(self, seq_id: int) -> int:
        return self._seq_len.get(seq_id, 0)

    def seq_n_blocks(self, seq_id: int) -> int:
        return len(self._seq_blocks.get(seq_id, ()))

    def extend_seq(self, seq_id: int, new_len: int) -> None:
        """Grow a sequence to new_len tokens, allocating blocks as needed."""
        blocks = self._seq_blocks[seq_id]
        need = (new_len + self.block_size - 1) // self.block_size
        while len(blocks) < need:
            if not self._free:
                raise RuntimeError(
                    f"KV pool exhausted ({self.n_blocks} blocks of {self.block_size})"
                )
            blocks.append(self._free.pop())
        self._seq_len[seq_id] = new_len

    def slot_mapping(self, seq_id: int, positions: Sequence[int]) -> List[int]:
        blocks = self._seq_blocks[seq_id]
        return [
            blocks[p // self.block_size] * self.block_size + p % self.block_size
            for p in positions
        ]

    def block_table(self, seq_ids: Sequence[int]) -> torch.Tensor:
        """Padded [B, max_blocks] int32 device tensor."""
        tables = [self._seq_blocks[s] for s in seq_ids]
        width = max(1, max(len(t) for t in tables))
        out = torch.zeros(len(tables), width, dtype=torch.int32)
        for i, t in enumerate(tables):
            if t:
                out[i, : len(t)] = torch.tensor(t, dtype=torch.int32)
        return out.to(self.device, non_blocking=True)
