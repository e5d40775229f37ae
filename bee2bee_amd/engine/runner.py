"""Runner: executes the transformer layer stack with bee2bee_amd.ops.

This is the replacement for the reference's `transformers.generate()` hot
loop (bee2bee/hf.py:84-108): explicit prefill/decode forwards over fused
weights, paged KV, and the HIP kernel set. Projection GEMMs go through
F.linear (hipBLASLt); everything fused is ops.* (HIP on GPU).

Pipeline parallelism: a Runner can own a contiguous layer range; the first
stage embeds tokens, the last stage applies the final norm + lm_head
(parallel/pp.py moves the hidden states between stages over RCCL).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from .. import ops
from ..models.spec import ModelSpec
from ..models.weights import ModelWeights
from .kv import PagedKV


class Runner:
    def __init__(
        self,
        spec: ModelSpec,
        weights: ModelWeights,
        kv: PagedKV,
        device: torch.device,
        dtype: torch.dtype = torch.bfloat16,
        layer_range: Optional[Tuple[int, int]] = None,
    ) -> None:
        self.spec = spec
        self.weights = weights
        self.kv = kv
        self.device = device
        self.dtype = dtype
        self.layer_lo, self.layer_hi = layer_range or (0, spec.n_layers)
        self.scale = spec.head_dim**-0.5
        # optional expert parallelism (parallel/ep.py); when set, MoE layers
        # dispatch tokens over RCCL all-to-all to the expert owners
        self.ep = None
        # optional tensor parallelism (parallel/tp.py): weights are a
        # head/intermediate shard and the two row-parallel projections
        # all-reduce their partial outputs over RCCL
        self.tp_group = None
        self.decode_attn_fn = None  # CP hook (parallel/cp.py)
        # hybrid stacks: rotation tables per (dims, base) of their latent-
        # attention layers, and an optional per-layer probe
        # layer_tap(layer_idx, residual_fp32) for bring-up/debugging
        self._rope_by_cfg = {}
        self._zeros = {}        # fp32 zero vectors by length (zero-logit sinks)
        self.layer_tap = None
        if spec.is_hybrid:
            self.rope_cos = self.rope_sin = None
            return
        cos, sin = ops.rope_tables(
            spec.max_seq_len, spec.head_dim, spec.rope_theta, device,
            scaling=spec.rope_scaling,
        )
        self.rope_cos, self.rope_sin = cos, sin

    @property
    def is_first_stage(self) -> bool:
        return self.layer_lo == 0

    @property
    def is_last_stage(self) -> bool:
        return self.layer_hi == self.spec.n_layers

    # ------------------------------------------------------------- forwards

    def embed(self, input_ids: torch.Tensor,
              positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        h = F.embedding(input_ids, self.weights.embed)
        if self.spec.pos_type == "learned" and positions is not None:
            h = h + F.embedding(positions.long(), self.weights.pos_embed)
        return h

    def _norm(self, x, w, b):
        if self.spec.norm_type == "layernorm":
            return ops.layernorm(x, w, b, self.spec.rms_eps)
        return ops.rmsnorm(x, w, self.spec.rms_eps)

    def _fused_add_norm(self, x, resid, w, b):
        if self.spec.norm_type == "layernorm":
            return ops.fused_add_layernorm(x, resid, w, b, self.spec.rms_eps)
        return ops.fused_add_rmsnorm(x, resid, w, self.spec.rms_eps)

    def lm_head(self, hidden: torch.Tensor) -> torch.Tensor:
        if self.spec.is_hybrid and self.spec.norm_type == "group_rmsnorm":
            # fp32 residual stream, weighted grouped final norm
            normed = ops.add_group_rmsnorm(
                hidden.contiguous(), None, None, None,
                self.weights.final_norm, self.spec.norm_groups,
                self.spec.rms_eps, self.dtype)
            return F.linear(normed, self.weights.lm_head)
        if self.spec.is_hybrid and self.weights.final_gain is None:
            # fp32 residual stream, weighted final norm
            normed = ops.rmsnorm_f32(
                hidden.contiguous(), self.weights.final_norm,
                self.spec.rms_eps, self.dtype)
            return F.linear(normed, self.weights.lm_head)
        if self.spec.is_hybrid:
            # hidden is the fp32 residual stream; scalar-gain final norm
            normed = ops.scalar_rmsnorm(
                hidden.contiguous(), self.weights.final_gain,
                self.spec.rms_eps, self.dtype)
            return F.linear(normed, self.weights.lm_head)
        normed = self._norm(hidden, self.weights.final_norm,
                            self.weights.final_norm_bias)
        return F.linear(normed, self.weights.lm_head)

    def _layer(
        self,
        layer_idx: int,
        hidden: torch.Tensor,
        residual: Optional[torch.Tensor],
        positions: torch.Tensor,
        slot_mapping: torch.Tensor,
        attn_fn,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        s = self.spec
        lw = self.weights.layers[layer_idx]
        if residual is None:
            residual = hidden
            normed = self._norm(hidden, lw.attn_norm, lw.attn_norm_bias)
        else:
            normed, residual = self._fused_add_norm(
                hidden, residual, lw.attn_norm, lw.attn_norm_bias
            )

        qkv = F.linear(normed, lw.wqkv)  # column-parallel under TP
        if lw.wqkv_bias is not None:  # Qwen2-style attention bias
            qkv = qkv + lw.wqkv_bias
        T = qkv.shape[0]
        q, k, v = qkv.split([s.q_size, s.kv_size, s.kv_size], dim=-1)
        q = q.view(T, s.n_heads, s.head_dim)
        k = k.view(T, s.n_kv_heads, s.head_dim)
        v = v.view(T, s.n_kv_heads, s.head_dim)
        if s.pos_type == "rope":
            ops.rope_inplace(q, k, positions, self.rope_cos, self.rope_sin)
        k_cache, v_cache = self.kv.layer(layer_idx)
        ops.kv_cache_store(k, v, k_cache, v_cache, slot_mapping)
        attn_out = attn_fn(layer_idx, q, k, v, k_cache, v_cache)
        attn_out = F.linear(attn_out.reshape(T, s.q_size), lw.wo, lw.wo_bias)
        if self.tp_group is not None:
            # row-parallel o-projection: sum the per-shard partials
            import torch.distributed as dist

            dist.all_reduce(attn_out, group=self.tp_group)

        normed, residual = self._fused_add_norm(
            attn_out, residual, lw.mlp_norm, lw.mlp_norm_bias
        )
        if s.is_moe:
            mlp_out = self._moe_mlp(lw, normed)
        elif s.act_type == "gelu":
            fc = F.linear(normed, lw.w_gate_up, lw.w_gate_up_bias)
            mlp_out = F.linear(ops.gelu(fc), lw.w_down, lw.w_down_bias)
        else:
            gate_up = F.linear(normed, lw.w_gate_up)
            mlp_out = F.linear(ops.swiglu(gate_up), lw.w_down)
            if self.tp_group is not None:
                # row-parallel down-projection
                import torch.distributed as dist

                dist.all_reduce(mlp_out, group=self.tp_group)
        return mlp_out, residual

    # below this many tokens the MoE layer runs all experts densely: at
    # decode batch sizes every expert's weights stream from HBM anyway
    # (bandwidth-bound), a batched GEMM reads them exactly once with full
    # MFMA efficiency, and every shape is static -> hipGraph-capturable
    # (the per-expert gather loop was 768 tiny launches per Mixtral step)
    MOE_DENSE_MAX_TOKENS = 256
    # above the dense threshold: sort token-slots by expert and run the
    # grouped-GEMM HIP kernel per projection — weights read once per expert,
    # flops proportional to routed tokens, segment sizes stay on device
    # (static shapes -> graph-capturable, no host sync). The kernel
    # accumulates 128 rows per W pass, so it is the default while the
    # AVERAGE segment fits one pass (T*k <= E*128); bigger batches re-read
    # W per extra pass and the padded bmm wins — those sizes only occur on
    # the (uncaptured) prefill path, where the host sync is harmless.
    MOE_GROUPED_ROWS = 128
    MOE_BMM_MAX_TOKENS = 100_000

    @classmethod
    def moe_grouped_max_tokens(cls, spec) -> int:
        return cls.MOE_GROUPED_ROWS * spec.n_experts // spec.top_k_experts

    @staticmethod
    def moe_grouped_aligned(spec) -> bool:
        """grouped_gemm kernel dim constraints (N%64, K%128) for both
        projections: gate_up [2I, H] and down [H, I]."""
        h, i = spec.hidden_size, spec.intermediate_size
        return h % 128 == 0 and i % 128 == 0

    @classmethod
    def moe_graph_capturable(cls, spec, max_tokens: int) -> bool:
        """True when every decode bucket up to max_tokens takes a
        capture-safe MoE path (dense or grouped — never padded bmm)."""
        if max_tokens <= cls.MOE_DENSE_MAX_TOKENS:
            return True
        return (cls.moe_grouped_aligned(spec)
                and max_tokens <= cls.moe_grouped_max_tokens(spec))

    def _moe_mlp(self, lw, x: torch.Tensor, ffn=None) -> torch.Tensor:
        """Top-k expert MLP: dense all-experts bmm for decode-sized batches,
        per-expert gather/GEMM/scatter for prefill-sized ones.

        ffn (models/hybrid.py MoEFFNSpec) overrides the uniform-stack
        sizes per layer, routes on fp32 logits and applies the layer's
        activation (clamped GLU or silu GLU) and scoring rule (softmax over
        the chosen logits, or softmax over all experts with a group-limited
        choice); the three execution strategies are shared."""
        s = self.spec
        if ffn is not None:
            E, I, top_k = ffn.n_experts, ffn.ff, ffn.top_k
            logits = F.linear(x.float(), lw.moe_gate)

            def act_fn(gu):
                if ffn.act == "silu_glu":
                    return ops.silu_glu(gu)
                if ffn.act == "gelu":
                    return ops.gelu_erf(gu)
                return ops.clamped_glu(gu, ffn.limit, ffn.alpha)
        else:
            E, I, top_k = s.n_experts, s.intermediate_size, s.top_k_experts
            act_fn = ops.swiglu
        # rows of an expert's input-side matrix: gate|up, or up alone
        U = lw.moe_w_gate_up.shape[1]
        if ffn is None and self.ep is not None:
            if self.weights.expert_range is not None:
                # weights hold only this rank's expert shard (EP sharding)
                w_gu, w_dn = lw.moe_w_gate_up, lw.moe_w_down
            else:
                lo = self.ep.e_lo
                hi = lo + self.ep.local_e
                w_gu, w_dn = lw.moe_w_gate_up[lo:hi], lw.moe_w_down[lo:hi]
            return self.ep.forward(x, lw.moe_gate, w_gu, w_dn)
        if ffn is None:
            logits = F.linear(x, lw.moe_gate)
        if ffn is not None and ffn.score in ("softmax_all", "sigmoid_all"):
            # scores over all experts, group-limited choice, no renorm
            weights, idx = ops.group_topk_gate(
                logits, top_k, ffn.n_groups, ffn.keep_groups,
                "sigmoid" if ffn.score == "sigmoid_all" else "softmax",
                ffn.group_top)
        else:
            weights, idx = ops.moe_topk_gate(logits, top_k)  # [T,k]
        T, H = x.shape

        if T <= self.MOE_DENSE_MAX_TOKENS:
            x_e = x.unsqueeze(0).expand(E, T, H)
            gu = torch.bmm(x_e, lw.moe_w_gate_up.transpose(1, 2))  # [E,T,2I]
            act = act_fn(gu.reshape(E * T, U)).view(E, T, I)
            y = torch.bmm(act, lw.moe_w_down.transpose(1, 2))  # [E,T,H]
            wfull = torch.zeros(T, E, dtype=torch.float32, device=x.device)
            wfull.scatter_(1, idx.long(), weights)
            out = torch.einsum("eth,te->th", y.float(), wfull)
            return out.to(x.dtype)

        import os as _os

        use_grouped = (
            x.device.type == "cuda"
            and x.dtype == torch.bfloat16  # the kernel's only instantiation
            and H % 128 == 0 and I % 128 == 0
            and T <= self.MOE_GROUPED_ROWS * E // top_k
            and _os.environ.get("BEE2BEE_MOE_BMM") != "1"
        )
        # the padded bmm stays CPU-only (and opt-in for A/B measurement):
        # hipBLASLt's batched TN bf16 kernel memory-faults on gfx950 once
        # the padded M reaches ~1K (repro: scripts/debug_moe_t4096.py, C
        # 1049 AND 1056) — GPU sizes above the grouped range take the
        # per-expert GEMM loop below, whose plain TN GEMMs are solid
        use_bmm = (x.device.type != "cuda"
                   or _os.environ.get("BEE2BEE_MOE_BMM") == "1")
        if T <= self.MOE_BMM_MAX_TOKENS and (use_grouped or use_bmm):
            # counting sort from one-hot cumsums: every op here (one_hot,
            # cumsum, gather, index_copy) is hipGraph-capture-safe —
            # torch.bincount/argsort are not
            k = top_k
            S = T * k
            flat_e = idx.reshape(-1).to(torch.int64)  # slot s -> expert
            oh = F.one_hot(flat_e, E)  # [S, E]
            counts = oh.sum(0)
            offs_excl = counts.cumsum(0) - counts
            rank = (oh.cumsum(0) - oh).gather(1, flat_e.unsqueeze(1)).squeeze(1)
            pos = (offs_excl[flat_e] + rank).to(torch.int64)  # dest row
            tok = torch.arange(S, device=x.device, dtype=torch.int64) // k
            if use_grouped:
                # grouped-GEMM HIP kernel (default in this range): no host
                # sync, static shapes -> the whole MoE decode step hipGraph-
                # captures; measured 3.8 TB/s of W per projection
                offsets = torch.zeros(E + 1, dtype=torch.int32, device=x.device)
                offsets[1:] = counts.cumsum(0).to(torch.int32)
                x_sorted = torch.empty(S, H, dtype=x.dtype, device=x.device)
                x_sorted.index_copy_(0, pos, x[tok])
                gu = ops.grouped_gemm(x_sorted, lw.moe_w_gate_up, offsets)
                act = act_fn(gu)
                y = ops.grouped_gemm(act, lw.moe_w_down, offsets)  # [S, H]
                contrib = y[pos].float()  # back to slot order
            else:
                # padded per-expert bmm: weights read once per expert, flops
                # proportional to max routed count; counts.max() is one host
                # sync per MoE layer (so no hipGraph above the dense range).
                # M aligns up to 16: odd M (e.g. 1049) faults hipBLASLt's
                # TN bf16 batched kernel on gfx950 (repro:
                # scripts/debug_moe_t4096.py; <2% padded flops)
                C = (int(counts.max()) + 15) & ~15
                padded = torch.zeros(E, C, H, dtype=x.dtype, device=x.device)
                padded[flat_e, rank] = x[tok]
                gu = torch.bmm(padded, lw.moe_w_gate_up.transpose(1, 2))
                act = act_fn(gu.reshape(E * C, U)).view(E, C, I)
                y = torch.bmm(act, lw.moe_w_down.transpose(1, 2))  # [E,C,H]
                contrib = y[flat_e, rank].float()  # [S, H] slot order
            out = torch.zeros(T, H, dtype=torch.float32, device=x.device)
            out.index_add_(
                0, tok, contrib * weights.reshape(-1).unsqueeze(-1)
            )
            return out.to(x.dtype)

        out = torch.zeros_like(x, dtype=torch.float32)
        for e in range(E):
            mask = idx == e  # [T, k]
            if not bool(mask.any()):
                continue
            tok, kslot = mask.nonzero(as_tuple=True)
            xe = x[tok]
            ge = F.linear(xe, lw.moe_w_gate_up[e])
            ye = F.linear(act_fn(ge), lw.moe_w_down[e])
            out.index_add_(0, tok, ye.float() * weights[tok, kslot, None])
        return out.to(x.dtype)

    def _run_layers(
        self,
        hidden: torch.Tensor,
        positions: torch.Tensor,
        slot_mapping: torch.Tensor,
        attn_fn,
    ) -> torch.Tensor:
        residual = None
        for layer_idx in range(self.layer_lo, self.layer_hi):
            hidden, residual = self._layer(
                layer_idx, hidden, residual, positions, slot_mapping, attn_fn
            )
        return hidden + residual if residual is not None else hidden

    def forward_prefill(
        self,
        input_ids_or_hidden: torch.Tensor,
        positions: torch.Tensor,
        slot_mapping: torch.Tensor,
        cu_seqlens: torch.Tensor,
        max_seqlen: int,
        block_table: Optional[torch.Tensor] = None,
        seq_lens: Optional[torch.Tensor] = None,
        query_lens: Optional[torch.Tensor] = None,
        state_slots: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """Full- or chunked-prompt forward. Returns final hidden [T, H]
        (call lm_head on the rows you need). When seq_lens/query_lens are
        given the chunk attends to the paged history (chunked prefill)."""
        if self.spec.is_hybrid:
            # hybrid stacks always attend through the pages and carry
            # per-sequence state; returns the fp32 residual stream
            return self._forward_hybrid(
                input_ids_or_hidden, positions, slot_mapping, cu_seqlens,
                max_seqlen, block_table, state_slots)
        chunked = seq_lens is not None

        def attn(layer_idx, q, k, v, k_cache, v_cache):
            if chunked:
                # chunked prefill: this chunk's K/V were just stored, so the
                # kernel reads K/V exclusively from the paged cache and masks
                # causally at absolute positions (HIP attn_prefill_mfma
                # <HD, PAGED=true>; reference attn_decode_with_history on CPU)
                return ops.attn_prefill_paged(
                    q, k_cache, v_cache, block_table, seq_lens, cu_seqlens,
                    max_seqlen, self.scale,
                )
            return ops.attn_prefill(q, k, v, cu_seqlens, max_seqlen, self.scale)

        hidden = (
            self.embed(input_ids_or_hidden, positions)
            if self.is_first_stage
            else input_ids_or_hidden
        )
        return self._run_layers(hidden, positions, slot_mapping, attn)

    def forward_decode(
        self,
        input_ids_or_hidden: torch.Tensor,
        positions: torch.Tensor,
        slot_mapping: torch.Tensor,
        block_table: torch.Tensor,
        seq_lens: torch.Tensor,
        state_slots: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """One-token-per-sequence step. input [B] ids (or [B, H] hidden for
        later pipeline stages); returns final hidden [B, H]."""
        if self.spec.is_hybrid:
            B = input_ids_or_hidden.shape[0]
            cu = torch.arange(B + 1, dtype=torch.int32, device=self.device)
            return self._forward_hybrid(
                input_ids_or_hidden, positions, slot_mapping, cu, 1,
                block_table, state_slots)

        def attn(layer_idx, q, k, v, k_cache, v_cache):
            if self.decode_attn_fn is not None:
                # injected attention (context parallelism: parallel/cp.py
                # merges per-rank partials over the local KV shard)
                return self.decode_attn_fn(
                    q, k_cache, v_cache, block_table, seq_lens, self.scale
                )
            return ops.attn_decode(
                q, k_cache, v_cache, block_table, seq_lens, self.scale
            )

        hidden = (
            self.embed(input_ids_or_hidden, positions)
            if self.is_first_stage
            else input_ids_or_hidden
        )
        return self._run_layers(hidden, positions, slot_mapping, attn)

    # --------------------------------------------------------- hybrid stacks

    def _rope_tables(self, dims: int, base: float, f64: bool = False,
                     scaling=None):
        """cos/sin tables per (dims, base[, scaling]); f64: angles evaluated
        in float64 before the single rounding to fp32. scaling: the
        wavelength-dependent frequency scaling {factor, original, fast,
        slow} (always float64 angles)."""
        key = (dims, base, f64,
               tuple(sorted(scaling.items())) if scaling else None)
        t = self._rope_by_cfg.get(key)
        if t is None:
            if scaling and "kind" in scaling:
                # linear or banded frequency scaling
                t = ops.rope_freq_tables(self.spec.max_seq_len, dims, base,
                                         scaling, self.device)
            elif scaling:
                t = ops.rope_tables_scaled(self.spec.max_seq_len, dims, base,
                                           scaling, self.device)
            else:
                make = ops.rope_tables_f64 if f64 else ops.rope_tables
                t = make(self.spec.max_seq_len, dims, base, self.device)
            self._rope_by_cfg[key] = t
        return t

    def _forward_hybrid(
        self,
        input_ids: torch.Tensor,
        positions: torch.Tensor,
        slot_mapping: torch.Tensor,
        cu_seqlens: torch.Tensor,
        max_qlen: int,
        block_table: torch.Tensor,
        state_slots: torch.Tensor,
    ) -> torch.Tensor:
        """One step of a hybrid stack over B packed chunks (prompt portions
        and single decode tokens alike). The residual stream is fp32
        end to end; each sublayer is normed before AND after:
            x += g_post * unit(mixer(conv(g_pre * unit(x))))
        and the post-norm + residual add + next pre-norm run as one fused
        kernel. Returns the fp32 residual [T, width]."""
        s, W = self.spec, self.weights
        if block_table is None or state_slots is None:
            raise ValueError("hybrid stacks need block_table and state_slots")
        T = input_ids.shape[0]
        B = cu_seqlens.shape[0] - 1
        if max_qlen == 1:
            seq_idx = cu_seqlens[:-1]
        else:
            lens = (cu_seqlens[1:] - cu_seqlens[:-1]).long()
            seq_idx = torch.repeat_interleave(
                torch.arange(B, dtype=torch.int32, device=self.device), lens,
                output_size=T)
        meta = (positions, slot_mapping, cu_seqlens, seq_idx, block_table,
                state_slots, max_qlen)
        x = F.embedding(input_ids, W.embed).float()
        if s.embed_scale != 1.0:
            x = x * s.embed_scale
        n = s.n_layers
        if s.layer_specs[0].form == "sandwich_w":
            return self._forward_sandwich_w(x, meta)
        if s.layer_specs[0].form == "parallel_gated":
            return self._forward_parallel_gated(x, meta)
        if s.layer_specs[0].form == "parallel":
            # x += mixer(h) + ffn(h), h = unit(x) * w: the residual add and
            # the next layer's norm run as one kernel
            eps, dt = s.rms_eps, self.dtype
            normed = ops.rmsnorm_f32(x, W.layers[0].norm_w, eps, dt)
            for i in range(n):
                y = self._parallel_layer(i, normed, meta)
                nxt = W.layers[i + 1].norm_w if i + 1 < n else None
                normed = ops.add_rmsnorm_f32(x, y, nxt, eps, dt)
                if self.layer_tap is not None:
                    self.layer_tap(i, x)
            return x
        normed = ops.scalar_rmsnorm(x, W.layers[0].gains[0], s.rms_eps,
                                    self.dtype)
        for i in range(n):
            nxt = W.layers[i + 1].gains[0] if i + 1 < n else None
            normed = self._hybrid_layer(i, x, normed, meta, nxt)
            if self.layer_tap is not None:
                self.layer_tap(i, x)
        return x

    def _hybrid_layer(self, i: int, x: torch.Tensor, normed: torch.Tensor,
                      meta, next_gain: Optional[float]):
        """Updates the residual x in place; returns the next sublayer's
        normed input (None after the last layer)."""
        s = self.spec
        lw, l = self.weights.layers[i], s.layer_specs[i]
        (positions, slot_mapping, cu, seq_idx, block_table, state_slots,
         max_qlen) = meta
        m, eps, dt = l.mixer, s.rms_eps, self.dtype
        T = normed.shape[0]
        h = normed
        if lw.canon is not None:
            h = ops.canon_conv(h, lw.canon, self.kv.conv_state[i], state_slots,
                               cu, seq_idx, positions)
        proj = F.linear(h, lw.wqkv)
        H = m.heads
        if m.kind == "latent_attention":
            D, R, C = m.dim, m.rot_dim, m.kv_rank
            q = proj[:, : m.q_size].view(T, H, D + R)
            kv = proj[:, m.q_size : m.q_size + m.cache_dim]
            gate = proj[:, m.q_size + m.cache_dim :]
            cache = self.kv.k_cache[i]
            cos, sin = self._rope_tables(m.rope_dims, m.rope_base)
            ops.latent_rope_store(q[..., D:], kv, lw.kv_norm, eps, C,
                                  m.rope_dims, positions, cos, sin, cache,
                                  slot_mapping)
            # absorbed form: fold the key up-projection into the query and
            # the value up-projection into the output, so attention runs on
            # the cached latent rows directly (one shared row per token)
            q_abs = torch.bmm(q[..., :D].transpose(0, 1), lw.w_uk)  # [H,T,C]
            lat = ops.latent_attn(q_abs, q[..., D:], gate, cache, block_table,
                                  positions, seq_idx, cu, m.window, m.scale,
                                  max_qlen)
            o = torch.bmm(lat, lw.w_uv)                          # [H,T,Dv]
            y = F.linear(o.transpose(0, 1).reshape(T, H * m.vdim), lw.wo)
        else:
            HD, HV = H * m.dim, H * m.vdim
            q = proj[:, :HD].view(T, H, m.dim)
            k = proj[:, HD : 2 * HD].view(T, H, m.dim)
            v = proj[:, 2 * HD : 2 * HD + HV].view(T, H, m.vdim)
            gate = proj[:, 2 * HD + HV :]
            o = ops.lightning_attn(q, k, v, lw.decay, self.kv.rec_state[i],
                                   state_slots, cu, positions, max_qlen)
            y = F.linear(ops.gated_rmsnorm(o, lw.out_norm, gate, eps, dt),
                         lw.wo)
        f = l.ffn
        if f is None:
            return ops.add_scalar_rmsnorm(x, y, lw.gains[1], next_gain, eps, dt)
        normed2 = ops.add_scalar_rmsnorm(x, y, lw.gains[1], lw.gains[2], eps,
                                         dt)
        y = self._moe_mlp(lw, normed2, ffn=f)
        y2 = None
        if f.shared_ff:
            gu = F.linear(normed2, lw.w_gate_up)
            y2 = F.linear(ops.clamped_glu(gu, f.shared_limit, f.alpha),
                          lw.w_down)
        return ops.add_scalar_rmsnorm(x, y, lw.gains[3], next_gain, eps, dt,
                                      y2=y2)

    # ---------------------------------------------- weighted-sandwich layers

    def _forward_sandwich_w(self, x: torch.Tensor, meta) -> torch.Tensor:
        """x += w1b * gnorm(mixer(w1 * gnorm(x))); x += w2b * gnorm(ffn(w2 *
        gnorm(x))) with grouped RMS norms; a layer run with `step_row` adds
        that row of the step table to the residual first. Post-norm,
        residual add, step add and the next pre-norm are ONE kernel. The
        layer list is the list of RUNS: a repeated block appears once per
        pass, sharing weights (LayerSpec.weights_of) but not pages."""
        s, W = self.spec, self.weights
        G, eps, dt = s.norm_groups, s.rms_eps, self.dtype
        n = s.n_layers

        def step_of(i):
            r = s.layer_specs[i].step_row if i < n else None
            return None if r is None else W.step_table[r]

        normed = ops.add_group_rmsnorm(x, None, None, step_of(0),
                                       W.layers[0].norms[0], G, eps, dt)
        for i in range(n):
            lw, l = W.layers[i], s.layer_specs[i]
            y = self._talk_attn_part(i, l.mixer, lw, normed, meta)
            nxt_w = W.layers[i + 1].norms[0] if i + 1 < n else None
            nxt_step = step_of(i + 1)
            tap = self.layer_tap is not None
            f = l.ffn
            if f is not None:
                normed = ops.add_group_rmsnorm(x, y, lw.norms[1], None,
                                               lw.norms[2], G, eps, dt)
                if getattr(f, "n_experts", 0):
                    y = self._moe_mlp(lw, normed, ffn=f)
                else:
                    z = F.linear(normed, lw.w_gate_up)
                    y = F.linear(ops.polynorm(z, lw.act_coef, eps, dt),
                                 lw.w_down)
                post = lw.norms[3]
            else:
                post = lw.norms[1]
            if tap:
                # the probe sees the residual before the next run's step
                ops.add_group_rmsnorm(x, y, post, None, None, G, eps, dt)
                self.layer_tap(i, x)
                normed = (ops.add_group_rmsnorm(x, None, None, nxt_step,
                                                nxt_w, G, eps, dt)
                          if nxt_w is not None else None)
            else:
                normed = ops.add_group_rmsnorm(x, y, post, nxt_step, nxt_w,
                                               G, eps, dt)
        return x

    def _talk_attn_part(self, i: int, m, lw, h: torch.Tensor,
                        meta) -> torch.Tensor:
        """Head-mixing windowed attention of layer run i on the normed
        input h: one fused projection [q | k | v | gate]; rotation, unit
        norm and page store in one kernel; attention + head mixing + gate;
        output projection."""
        (positions, slot_mapping, cu, seq_idx, block_table, _,
         max_qlen) = meta
        T = h.shape[0]
        proj = F.linear(h, lw.wqkv)
        nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        q = proj[:, :nq].view(T, m.heads, m.dim)
        k = proj[:, nq : nq + nk].view(T, m.kv_heads, m.dim)
        v = proj[:, nq + nk : nq + nk + nv].view(T, m.kv_heads, m.vdim)
        gate = proj[:, nq + nk + nv :]
        cos = sin = None
        if m.rope_dims:
            cos, sin = self._rope_tables(m.rope_dims, m.rope_base, f64=True,
                                         scaling=m.rope_scaling)
        k_cache, v_cache = self.kv.k_cache[i], self.kv.v_cache[i]
        # q leaves this rotated, unit-norm and times the score scale
        ops.rope_unit_store(q, k, v, self.spec.rms_eps, m.rope_dims,
                            positions, cos, sin, m.scale, k_cache, v_cache,
                            slot_mapping)
        out = torch.empty(T, m.out_size, dtype=self.dtype, device=h.device)
        ops.talk_attn(q, k_cache, v_cache, block_table, positions, seq_idx,
                      cu, lw.talk, gate, m.window, out, max_qlen)
        return F.linear(out, lw.wo)

    # ------------------------------------------ gated parallel-form layers

    def _forward_parallel_gated(self, x: torch.Tensor, meta) -> torch.Tensor:
        """x += sigmoid(g1) * mixer(h) + sigmoid(g2) * ffn(h) with h =
        unit(x) * w and both gates projections of h. The layer list is the
        list of RUNS (a repeated block appears once per pass, sharing
        weights but not pages or state); a run with `readd_embed` adds the
        embedding output to the residual first. The two gated adds, that
        add and the next run's norm are ONE kernel."""
        s, W = self.spec, self.weights
        eps, dt, n = s.rms_eps, self.dtype, s.n_layers
        e0 = x.clone() if any(l.readd_embed for l in s.layer_specs) else None
        normed = ops.rmsnorm_f32(x, W.layers[0].norm_w, eps, dt)
        for i in range(n):
            y1, g1, y2, g2 = self._gated_layer(i, normed, meta)
            nxt = W.layers[i + 1].norm_w if i + 1 < n else None
            extra = e0 if i + 1 < n and s.layer_specs[i + 1].readd_embed \
                else None
            if self.layer_tap is not None and extra is not None:
                # the probe sees the residual before the next pass's add
                ops.gated_add_rmsnorm(x, y1, g1, y2, g2, None, None, eps, dt)
                self.layer_tap(i, x)
                normed = ops.gated_add_rmsnorm(x, None, None, None, None,
                                               extra, nxt, eps, dt)
                continue
            normed = ops.gated_add_rmsnorm(x, y1, g1, y2, g2, extra, nxt,
                                           eps, dt)
            if self.layer_tap is not None:
                self.layer_tap(i, x)
        return x

    def _gated_layer(self, i: int, h: torch.Tensor, meta):
        """Sublayer outputs and raw gates of layer run i: (mixer(h), g1,
        ffn(h) or None, g2 or None). One input GEMM (with its bias vector)
        covers every projection that reads h, the gates included."""
        from ..models.hybrid import mixer_parts

        s = self.spec
        lw, l = self.weights.layers[i], s.layer_specs[i]
        ins, _ = lw.layout
        proj = F.linear(h, lw.w_in, lw.b_in)

        def cols(key):
            off, n = ins[key]
            return proj[:, off : off + n]

        m = l.mixer
        ys = []
        for pre, part in mixer_parts(m):
            ns = lw.mix[pre]
            if part.kind == "gqa_attention":
                o = self._gqa_attn_part(i, part, ns, cols, pre, meta)
            elif part.kind == "latent_attention":
                o = self._latent_attn_part(i, part, ns, cols, pre, meta)
            else:
                o = self._min_gru_part(i, part, cols, pre, meta)
            ys.append(F.linear(o, ns.wo, ns.wo_b))
        if m.kind == "parallel":
            if m.combine != "normed_mean":
                raise ValueError(f"unknown combine {m.combine!r}")
            y1 = ops.pair_rmsnorm_mean(
                ys[0], lw.mix["left."].out_norm, ys[1],
                lw.mix["right."].out_norm, s.rms_eps, self.dtype)
        else:
            y1 = ys[0]
        if l.ffn is None:
            return y1, cols("rg1"), None, None
        y2 = self._moe_mlp(lw, h, ffn=l.ffn)
        return y1, cols("rg1"), y2, cols("rg2")

    def _gqa_attn_part(self, i: int, m, ns, cols, pre, meta) -> torch.Tensor:
        """Grouped-query attention of layer run i: optional short conv on
        the projected q|k|v (fp32 out), rotation + page store, attention
        with the spec's cap / score mix / sink / window / head gate."""
        (positions, slot_mapping, cu, seq_idx, block_table, state_slots,
         max_qlen) = meta
        T = positions.shape[0]
        nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        off = cols(pre + "q")
        qkv = off.as_strided((T, nq + nk + nv), off.stride())
        if ns.conv_w is not None:
            conv_state = self.kv.conv_state[i]
            if conv_state is None:       # a single tap carries nothing
                conv_state = qkv.new_empty(0)
            qkv = ops.short_conv(qkv, ns.conv_w, conv_state, state_slots, cu,
                                 seq_idx, positions, False)
        q = qkv[:, :nq].view(T, m.heads, m.dim)
        k = qkv[:, nq : nq + nk].view(T, m.kv_heads, m.dim)
        v = qkv[:, nq + nk :].view(T, m.kv_heads, m.vdim)
        cos = sin = None
        if m.rope_dims:
            cos, sin = self._rope_tables(m.rope_dims, m.rope_base, f64=True,
                                         scaling=m.rope_scaling)
        k_cache, v_cache = self.kv.k_cache[i], self.kv.v_cache[i]
        # the query leaves this rotated and times the score scale
        if q.dtype == self.dtype:
            q_out = q
        else:
            q_out = torch.empty(T, m.heads, m.dim, dtype=self.dtype,
                                device=q.device)
        ops.rope_store(q, k, v, q_out, m.rope_dims,
                       m.rope_layout == "interleaved", positions, cos, sin,
                       m.scale, k_cache, v_cache, slot_mapping)
        sink = None
        if m.zero_sink:
            sink = self._zeros_f32(m.heads)
        out = torch.empty(T, m.out_size, dtype=self.dtype, device=q.device)
        ops.gqa_attn(q_out, k_cache, v_cache, block_table, positions, seq_idx,
                     cu, m.softcap, ns.talk if m.score_mix else None, sink,
                     cols(pre + "g") if m.head_gate else None, m.window, out,
                     max_qlen)
        return out

    def _zeros_f32(self, n: int) -> torch.Tensor:
        z = self._zeros.get(n)
        if z is None:
            z = self._zeros[n] = torch.zeros(n, dtype=torch.float32,
                                             device=self.device)
        return z

    def _latent_attn_part(self, i: int, m, ns, cols, pre, meta
                          ) -> torch.Tensor:
        """Latent attention of layer run i in absorbed form (the key
        up-projection folded into the query, the value up-projection into
        the output), queries through their own normed latent when the spec
        has one, a per-head sink and sigmoid head gate in the kernel."""
        (positions, slot_mapping, cu, seq_idx, block_table, _,
         max_qlen) = meta
        T, H = positions.shape[0], m.heads
        D, R, C = m.dim, m.rot_dim, m.kv_rank
        if m.q_rank:
            cq = ops.slice_rmsnorm(cols(pre + "dq"), ns.q_norm,
                                   self.spec.rms_eps)
            q = F.linear(cq, ns.w_uq).view(T, H, D + R)
        else:
            q = cols(pre + "q").view(T, H, D + R)
        kv, gate = cols(pre + "dkv"), cols(pre + "g")
        cache = self.kv.k_cache[i]
        cos, sin = self._rope_tables(m.rope_dims, m.rope_base, f64=True)
        ops.latent_rope_store(q[..., D:], kv, ns.kv_norm, self.spec.rms_eps,
                              C, m.rope_dims, positions, cos, sin, cache,
                              slot_mapping)
        q_abs = torch.bmm(q[..., :D].transpose(0, 1), ns.w_uk)    # [H,T,C]
        lat = ops.latent_attn(q_abs, q[..., D:], gate, cache, block_table,
                              positions, seq_idx, cu, m.window, m.scale,
                              max_qlen, sink=ns.sink)
        o = torch.bmm(lat, ns.w_uv)                              # [H,T,Dv]
        return o.transpose(0, 1).reshape(T, H * m.vdim)

    def _min_gru_part(self, i: int, m, cols, pre, meta) -> torch.Tensor:
        positions, _, cu, _, _, state_slots, max_qlen = meta
        T = positions.shape[0]
        out = torch.empty(T, m.width, dtype=self.dtype,
                          device=positions.device)
        ops.min_gru(cols(pre + "z"), cols(pre + "x"), cols(pre + "g"),
                    self.kv.rec_state[i], state_slots, cu, positions, out,
                    max_qlen)
        return out

    # ------------------------------------------------- parallel-form layers

    def _parallel_layer(self, i: int, h: torch.Tensor, meta) -> torch.Tensor:
        """mixer(h) + ffn(h) of layer i as two GEMMs: one input projection
        for everything that reads h (the feed-forward's up included), the
        mixer kernels and the activation writing column slices of ONE
        buffer, and one output projection over that buffer, which sums the
        mixer parts and the feed-forward in its fp32 accumulator."""
        from ..models.hybrid import mixer_parts

        s = self.spec
        lw, l = self.weights.layers[i], s.layer_specs[i]
        ins, n_in, outs, n_out = lw.layout
        T = h.shape[0]
        proj = F.linear(h, lw.w_in)                         # [T, n_in]
        exact = n_out == sum(n for _, n in outs.values())
        buf = (torch.empty if exact else torch.zeros)(
            T, n_out, dtype=self.dtype, device=h.device)

        def cols(key):
            off, n = ins[key]
            return proj[:, off : off + n]

        m = l.mixer
        for pre, part in mixer_parts(m):
            scale = 1.0
            if m.kind == "parallel":
                scale = m.left_scale if pre == "left." else m.right_scale
            off, n = outs[pre + "o"]
            out = buf[:, off : off + n]
            ns = lw.mix[pre]
            if part.kind == "retention":
                self._retention_part(i, part, ns, cols, pre, meta, out, scale)
            elif part.kind == "delta":
                self._delta_part(i, part, ns, cols, pre, meta, out, scale)
            else:
                self._sink_attn_part(i, part, ns, cols, pre, meta, out, scale)
        if l.ffn is not None:
            off, n = outs["down"]
            ops.relu2(cols("up"), buf[:, off : off + n])
        return F.linear(buf, lw.w_out)

    def _retention_part(self, i, m, ns, cols, pre, meta, out, scale) -> None:
        positions, _, cu, _, _, state_slots, max_qlen = meta
        T, H = positions.shape[0], m.heads
        cos = sin = None
        if m.rope_dims:
            cos, sin = self._rope_tables(m.rope_dims, m.rope_base, f64=True)
        o = ops.retention_attn(
            cols(pre + "q").view(T, H, m.dim), cols(pre + "k").view(T, H, m.dim),
            cols(pre + "v").view(T, H, m.vdim), ns.decay, m.rope_dims, cos,
            sin, m.dim ** -0.5, self.kv.rec_state[i], state_slots, cu,
            positions, max_qlen)
        ops.head_gated_norm(o.view(T, H, m.vdim), None, cols(pre + "g"),
                            "silu", self.spec.rms_eps, out, scale)

    def _delta_part(self, i, m, ns, cols, pre, meta, out, scale) -> None:
        positions, _, cu, seq_idx, _, state_slots, _ = meta
        T, H, G, D = positions.shape[0], m.heads, m.kv_heads, m.dim
        conv_state = self.kv.conv_state[i]
        if conv_state is None:       # a single tap carries nothing
            conv_state = out.new_empty(0)
        qkv = ops.short_conv(cols(pre + "qkv"), ns.conv_w, conv_state,
                             state_slots, cu, seq_idx, positions, True)
        a = cols(pre + "a")
        if ns.a2 is not None:
            a = F.linear(a, ns.a2)
        beta, g = ops.delta_gates(qkv, G, D, cols(pre + "b"), a, ns.dt_bias,
                                  ns.rate, m.channel_decay)
        nq = G * D
        o = ops.delta_rule(
            qkv[:, :nq].view(T, G, D), qkv[:, nq : 2 * nq].view(T, G, D),
            qkv[:, 2 * nq :].view(T, H, m.vdim), beta, g,
            self.kv.rec_state[i], state_slots, cu, positions)
        gate = cols(pre + "g")
        if ns.g2 is not None:
            gate = F.linear(gate, ns.g2)
        ops.head_gated_norm(o, ns.norm, gate, m.gate, self.spec.rms_eps, out,
                            scale)

    def _sink_attn_part(self, i, m, ns, cols, pre, meta, out, scale) -> None:
        (positions, slot_mapping, cu, seq_idx, block_table, _,
         max_qlen) = meta
        T = positions.shape[0]
        q = cols(pre + "q").view(T, m.heads, m.dim)
        k = cols(pre + "k").view(T, m.kv_heads, m.dim)
        cos = sin = None
        if m.rope_dims:
            cos, sin = self._rope_tables(m.rope_dims, m.rope_base, f64=True)
        k_cache, v_cache = self.kv.k_cache[i], self.kv.v_cache[i]
        # q leaves this with every score multiplier folded in
        ops.qk_norm_rope_store(q, k, ns.q_norm, ns.k_norm, self.spec.rms_eps,
                               m.rope_dims, positions, cos, sin, ns.q_mult,
                               k_cache, v_cache, slot_mapping)
        ops.sink_attn(q, k_cache, v_cache, block_table, positions, seq_idx,
                      cu, ns.sink, m.window, out, scale, max_qlen)
