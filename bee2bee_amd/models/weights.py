"""Model weights: HF-checkpoint-compatible loading (safetensors) and random
init — laid out the way the MI355X engine consumes them.

Engine layout decisions (MI355X-first):
  * qkv is fused into one [q+2kv, hidden] matrix and gate|up into one
    [2*inter, hidden] matrix per layer → one hipBLASLt GEMM each instead of
    three/two (fewer, larger GEMMs saturate MFMA and HBM better).
  * Weights live in bf16 on-device; 288 GB HBM3E holds Llama-3-70B (140 GB)
    on a single GPU with room for KV cache, so sharding is a choice
    (pipeline parallel), not a requirement.

HF name mapping (checkpoint compatibility, reference loads the same files via
transformers — bee2bee/hf.py:23-32):
  model.embed_tokens.weight, model.layers.{i}.self_attn.{q,k,v,o}_proj.weight,
  model.layers.{i}.mlp.{gate,up,down}_proj.weight,
  model.layers.{i}.{input,post_attention}_layernorm.weight, model.norm.weight,
  lm_head.weight; Mixtral: model.layers.{i}.block_sparse_moe.gate.weight and
  .experts.{e}.w{1,2,3}.weight.
"""
from __future__ import annotations

import glob
import json
import os
from typing import Dict, Iterator, Optional, Tuple

import torch

from .spec import ModelSpec


class LayerWeights:
    __slots__ = (
        "attn_norm", "attn_norm_bias", "wqkv", "wqkv_bias", "wo", "wo_bias",
        "mlp_norm", "mlp_norm_bias",
        "w_gate_up", "w_gate_up_bias", "w_down", "w_down_bias",  # dense mlp
        "moe_gate", "moe_w_gate_up", "moe_w_down",  # moe
        # hybrid stacks (models/hybrid.py): scalar norm gains, the input
        # conv, the latent attention's norm / up-projections, the linear
        # attention's output norm and per-head decay
        "gains", "canon", "kv_norm", "w_uk", "w_uv", "out_norm", "decay",
        # parallel-form layers: weighted norm, the two fused GEMMs (input
        # projections incl. the feed-forward's up; mixer outputs + down),
        # their column layouts, and the mixer parts' small fp32 tensors
        "norm_w", "w_in", "w_out", "layout", "mix",
        # weighted-sandwich layers: the four grouped-norm weights, the
        # attention's head-mixing matrix, the dense activation's numbers
        "norms", "talk", "act_coef",
        # gated parallel-form layers: the bias of the fused input matrix
        "b_in",
    )

    def __init__(self) -> None:
        self.attn_norm = None
        self.attn_norm_bias = None  # layernorm arch (gpt2)
        self.wqkv = None
        self.wqkv_bias = None  # Qwen2/gpt2 fused [q+2kv] bias (optional)
        self.wo = None
        self.wo_bias = None
        self.mlp_norm = None
        self.mlp_norm_bias = None
        self.w_gate_up = None       # gelu arch: the single fc [I, H]
        self.w_gate_up_bias = None
        self.w_down = None
        self.w_down_bias = None
        self.moe_gate = None
        self.moe_w_gate_up = None
        self.moe_w_down = None
        self.gains = None      # (pre-mixer, post-mixer, pre-ffn, post-ffn)
        self.canon = None      # [taps, width] fp32 (tap-major)
        self.kv_norm = None    # [kv_rank] fp32
        self.w_uk = None       # [heads, dim, kv_rank]
        self.w_uv = None       # [heads, kv_rank, vdim]
        self.out_norm = None   # [heads * vdim] fp32
        self.decay = None      # [heads] fp32
        self.norm_w = None     # [width] fp32
        self.w_in = None       # [in_total, width]
        self.w_out = None      # [width, out_total]
        self.layout = None     # models/hybrid.py fused_layout(layer)
        self.mix = None        # {part prefix: SimpleNamespace of tensors}
        self.norms = None      # 4 x [width] fp32: pre/post mixer, pre/post ffn
        self.talk = None       # [heads, heads] fp32
        self.act_coef = None   # [4] fp32 (PolyNorm a, b, c, e)
        self.b_in = None       # [in_total] (zeros where a part has no bias)


class ModelWeights:
    def __init__(self, spec: ModelSpec, device: torch.device, dtype: torch.dtype) -> None:
        self.spec = spec
        self.device = device
        self.dtype = dtype
        self.embed: Optional[torch.Tensor] = None  # [vocab, hidden]
        self.pos_embed: Optional[torch.Tensor] = None  # [max_seq, hidden]
        self.final_norm: Optional[torch.Tensor] = None  # [hidden]
        self.final_norm_bias: Optional[torch.Tensor] = None
        self.lm_head: Optional[torch.Tensor] = None  # [vocab, hidden]
        self.final_gain: Optional[float] = None  # scalar-gain final norm
        self.step_table: Optional[torch.Tensor] = None  # [passes, hidden] fp32
        self.layers = [LayerWeights() for _ in range(spec.n_layers)]
        # expert-parallel shard: when set, MoE expert tensors hold only
        # experts [lo, hi) (gate stays replicated); see parallel/ep.py
        self.expert_range: Optional[Tuple[int, int]] = None

    # -------------------------------------------------------------- random

    @torch.no_grad()
    def random_init(
        self,
        seed: int = 0,
        layer_range: Optional[Tuple[int, int]] = None,
        expert_range: Optional[Tuple[int, int]] = None,
    ) -> "ModelWeights":
        """Random weights of the real architecture (synthetic serving — the
        benchmark contract requires random-init weights of the named model).

        layer_range (for pipeline stages): only materialize layers [lo, hi);
        embed only on the first stage, head/final norm only on the last.
        expert_range (for expert parallelism): only materialize that expert
        shard — drawn per expert, so a shard holds exactly the values the
        full init would (EP-vs-single equivalence tests rely on this)."""
        s = self.spec
        if s.is_hybrid:
            if layer_range or expert_range:
                raise NotImplementedError(
                    "hybrid stacks are not sharded (pipeline/expert ranges)")
            if s.arch == "pugozen":
                return self._random_init_pugozen(seed)
            if s.arch == "pimodra":
                return self._random_init_pimodra(seed)
            if s.arch == "zevilorn":
                return self._random_init_zevilorn(seed)
            return self._random_init_hybrid(seed)
        lo, hi = layer_range or (0, s.n_layers)
        self.expert_range = expert_range
        e_lo, e_hi = expert_range or (0, getattr(s, "n_experts", 0) or 0)
        import zlib

        # Generate directly on the target device (an 8B randn on host would
        # serialize startup). Each tensor gets its own generator seeded by
        # (seed, tensor name) so a pipeline stage materializing only layers
        # [lo, hi) draws IDENTICAL values to a full single-process init —
        # the PP-vs-single-process equivalence tests rely on this.
        def rnd(name: str, *shape: int, std: float) -> torch.Tensor:
            tseed = (seed * 1000003 + zlib.crc32(name.encode())) % (2**31)
            gen = torch.Generator(device=self.device).manual_seed(tseed)
            t = torch.randn(*shape, generator=gen, dtype=torch.float32,
                            device=self.device)
            return (t * std).to(self.dtype)

        std = 0.02
        proj_std = std / max(1.0, (2 * s.n_layers) ** 0.5)
        zeros = lambda *shape: torch.zeros(  # noqa: E731
            *shape, device=self.device, dtype=self.dtype)
        if lo == 0:
            self.embed = rnd("embed", s.vocab_size, s.hidden_size, std=std)
            if s.pos_type == "learned":
                self.pos_embed = rnd("pos_embed", s.max_seq_len,
                                     s.hidden_size, std=0.01)
        if hi == s.n_layers:
            self.final_norm = torch.ones(
                s.hidden_size, device=self.device, dtype=self.dtype
            )
            if s.norm_type == "layernorm":
                self.final_norm_bias = zeros(s.hidden_size)
            if s.tie_embeddings:
                self.lm_head = (
                    self.embed
                    if self.embed is not None
                    else rnd("embed", s.vocab_size, s.hidden_size, std=std)
                )
            else:
                self.lm_head = rnd("lm_head", s.vocab_size, s.hidden_size, std=std)
        for i in range(lo, hi):
            lw = self.layers[i]
            lw.attn_norm = torch.ones(s.hidden_size, device=self.device, dtype=self.dtype)
            lw.mlp_norm = torch.ones(s.hidden_size, device=self.device, dtype=self.dtype)
            lw.wqkv = rnd(f"l{i}.wqkv", s.q_size + 2 * s.kv_size, s.hidden_size, std=std)
            if s.qkv_bias:
                lw.wqkv_bias = rnd(
                    f"l{i}.wqkv_b", s.q_size + 2 * s.kv_size, std=std
                )
            if s.norm_type == "layernorm":
                lw.attn_norm_bias = zeros(s.hidden_size)
                lw.mlp_norm_bias = zeros(s.hidden_size)
            lw.wo = rnd(f"l{i}.wo", s.hidden_size, s.q_size, std=proj_std)
            if s.attn_out_bias:
                lw.wo_bias = zeros(s.hidden_size)
            if s.is_moe:
                lw.moe_gate = rnd(f"l{i}.gate", s.n_experts, s.hidden_size, std=std)
                lw.moe_w_gate_up = torch.stack([
                    rnd(f"l{i}.w_gu.e{e}", 2 * s.intermediate_size,
                        s.hidden_size, std=std)
                    for e in range(e_lo, e_hi)
                ])
                lw.moe_w_down = torch.stack([
                    rnd(f"l{i}.w_dn.e{e}", s.hidden_size,
                        s.intermediate_size, std=proj_std)
                    for e in range(e_lo, e_hi)
                ])
            elif s.act_type == "gelu":
                lw.w_gate_up = rnd(f"l{i}.w_fc", s.intermediate_size,
                                   s.hidden_size, std=std)
                lw.w_down = rnd(f"l{i}.w_dn", s.hidden_size,
                                s.intermediate_size, std=proj_std)
                if s.mlp_bias:
                    lw.w_gate_up_bias = zeros(s.intermediate_size)
                    lw.w_down_bias = zeros(s.hidden_size)
            else:
                lw.w_gate_up = rnd(f"l{i}.w_gu", 2 * s.intermediate_size, s.hidden_size, std=std)
                lw.w_down = rnd(f"l{i}.w_dn", s.hidden_size, s.intermediate_size, std=proj_std)
        return self

    # ---------------------------------------------------------- safetensors

    @torch.no_grad()
    def load_hf(
        self,
        model_path: str,
        layer_range: Optional[Tuple[int, int]] = None,
        expert_range: Optional[Tuple[int, int]] = None,
    ) -> "ModelWeights":
        """Load HF safetensors shards, fusing qkv / gate|up on the fly.
        expert_range: keep only that expert shard on device (EP ranks)."""
        s = self.spec
        if s.is_hybrid:
            if layer_range or expert_range:
                raise NotImplementedError(
                    "hybrid stacks are not sharded (pipeline/expert ranges)")
            if s.arch == "pugozen":
                return self._load_pugozen(model_path)
            if s.arch == "pimodra":
                return self._load_pimodra(model_path)
            if s.arch == "zevilorn":
                return self._load_zevilorn(model_path)
            return self._load_nukopel(model_path)
        if s.arch == "gpt2":
            return self._load_gpt2(model_path, layer_range)
        lo, hi = layer_range or (0, s.n_layers)
        self.expert_range = expert_range
        e_lo, e_hi = expert_range or (0, getattr(s, "n_experts", 0) or 0)
        n_local_e = e_hi - e_lo
        want_embed = lo == 0
        want_head = hi == s.n_layers

        pending: Dict[str, Dict[str, torch.Tensor]] = {}

        def to_dev(t: torch.Tensor) -> torch.Tensor:
            return t.to(self.device, self.dtype, non_blocking=True)

        def try_fuse(i: int) -> None:
            lw = self.layers[i]
            p = pending.get(f"attn.{i}")
            if p and len(p) == 3 and lw.wqkv is None:
                lw.wqkv = torch.cat([p["q"], p["k"], p["v"]], dim=0)
                pending.pop(f"attn.{i}")
            p = pending.get(f"attnb.{i}")
            if p and len(p) == 3 and lw.wqkv_bias is None:
                lw.wqkv_bias = torch.cat([p["q"], p["k"], p["v"]], dim=0)
                pending.pop(f"attnb.{i}")
            p = pending.get(f"mlp.{i}")
            if p and len(p) == 2 and lw.w_gate_up is None:
                lw.w_gate_up = torch.cat([p["gate"], p["up"]], dim=0)
                pending.pop(f"mlp.{i}")

        for name, tensor in iter_safetensors(model_path):
            parts = name.split(".")
            if name == "model.embed_tokens.weight":
                if want_embed:
                    self.embed = to_dev(tensor)
                elif want_head and s.tie_embeddings:
                    # PP LAST stage of a tied checkpoint: the head IS the
                    # embedding matrix, which only ships as embed_tokens
                    self.lm_head = to_dev(tensor)
                continue
            if name == "model.norm.weight":
                if want_head:
                    self.final_norm = to_dev(tensor)
                continue
            if name == "lm_head.weight":
                if want_head:
                    self.lm_head = to_dev(tensor)
                continue
            if len(parts) < 4 or parts[0] != "model" or parts[1] != "layers":
                continue
            i = int(parts[2])
            if not (lo <= i < hi):
                continue
            lw = self.layers[i]
            sub = ".".join(parts[3:])
            if sub == "input_layernorm.weight":
                lw.attn_norm = to_dev(tensor)
            elif sub == "post_attention_layernorm.weight":
                lw.mlp_norm = to_dev(tensor)
            elif sub == "self_attn.q_proj.weight":
                pending.setdefault(f"attn.{i}", {})["q"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "self_attn.k_proj.weight":
                pending.setdefault(f"attn.{i}", {})["k"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "self_attn.v_proj.weight":
                pending.setdefault(f"attn.{i}", {})["v"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "self_attn.q_proj.bias":
                pending.setdefault(f"attnb.{i}", {})["q"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "self_attn.k_proj.bias":
                pending.setdefault(f"attnb.{i}", {})["k"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "self_attn.v_proj.bias":
                pending.setdefault(f"attnb.{i}", {})["v"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "self_attn.o_proj.weight":
                lw.wo = to_dev(tensor)
            elif sub == "mlp.gate_proj.weight":
                pending.setdefault(f"mlp.{i}", {})["gate"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "mlp.up_proj.weight":
                pending.setdefault(f"mlp.{i}", {})["up"] = to_dev(tensor)
                try_fuse(i)
            elif sub == "mlp.down_proj.weight":
                lw.w_down = to_dev(tensor)
            elif sub == "block_sparse_moe.gate.weight":
                lw.moe_gate = to_dev(tensor)
            elif parts[3] == "block_sparse_moe" and parts[4] == "experts":
                e = int(parts[5])
                if not (e_lo <= e < e_hi):
                    continue  # expert owned by another EP rank
                w = parts[6]  # w1 (gate), w2 (down), w3 (up)
                key = f"moe.{i}"
                pending.setdefault(key, {})[f"{w}.{e}"] = to_dev(tensor)
                p = pending[key]
                if len(p) == 3 * n_local_e:
                    lw.moe_w_gate_up = torch.stack(
                        [
                            torch.cat([p[f"w1.{e2}"], p[f"w3.{e2}"]], dim=0)
                            for e2 in range(e_lo, e_hi)
                        ]
                    )
                    lw.moe_w_down = torch.stack(
                        [p[f"w2.{e2}"] for e2 in range(e_lo, e_hi)]
                    )
                    pending.pop(key)

        if want_head and self.lm_head is None:
            # tied embeddings checkpoints omit lm_head
            self.lm_head = self.embed
        missing = []
        if want_embed and self.embed is None:
            missing.append("embed_tokens")
        for i in range(lo, hi):
            if self.layers[i].wqkv is None:
                missing.append(f"layers.{i}.qkv")
        if missing:
            raise FileNotFoundError(
                f"checkpoint at {model_path} is missing tensors: {missing[:5]}"
            )
        return self


    @torch.no_grad()
    def _load_gpt2(self, model_path: str,
                   layer_range: Optional[Tuple[int, int]] = None
                   ) -> "ModelWeights":
        """GPT-2 family safetensors (wte/wpe/h.N.*): Conv1D weights are
        stored transposed ([in, out]) and qkv ships pre-fused as c_attn."""
        s = self.spec
        lo, hi = layer_range or (0, s.n_layers)

        def to_dev(t: torch.Tensor) -> torch.Tensor:
            return t.to(self.device, self.dtype, non_blocking=True)

        for name, tensor in iter_safetensors(model_path):
            name = name[len("transformer."):] if name.startswith(
                "transformer.") else name
            if name == "wte.weight":
                if lo == 0:
                    self.embed = to_dev(tensor)
                elif hi == s.n_layers:
                    self.lm_head = to_dev(tensor)  # tied head, PP last stage
                continue
            if name == "wpe.weight":
                if lo == 0:
                    self.pos_embed = to_dev(tensor)
                continue
            if name == "ln_f.weight":
                if hi == s.n_layers:
                    self.final_norm = to_dev(tensor)
                continue
            if name == "ln_f.bias":
                if hi == s.n_layers:
                    self.final_norm_bias = to_dev(tensor)
                continue
            parts = name.split(".")
            if parts[0] != "h":
                continue
            i = int(parts[1])
            if not (lo <= i < hi):
                continue
            lw = self.layers[i]
            rest = ".".join(parts[2:])
            if rest == "ln_1.weight":
                lw.attn_norm = to_dev(tensor)
            elif rest == "ln_1.bias":
                lw.attn_norm_bias = to_dev(tensor)
            elif rest == "ln_2.weight":
                lw.mlp_norm = to_dev(tensor)
            elif rest == "ln_2.bias":
                lw.mlp_norm_bias = to_dev(tensor)
            elif rest == "attn.c_attn.weight":
                lw.wqkv = to_dev(tensor.t().contiguous())  # Conv1D -> [3H, H]
            elif rest == "attn.c_attn.bias":
                lw.wqkv_bias = to_dev(tensor)
            elif rest == "attn.c_proj.weight":
                lw.wo = to_dev(tensor.t().contiguous())
            elif rest == "attn.c_proj.bias":
                lw.wo_bias = to_dev(tensor)
            elif rest == "mlp.c_fc.weight":
                lw.w_gate_up = to_dev(tensor.t().contiguous())  # [I, H]
            elif rest == "mlp.c_fc.bias":
                lw.w_gate_up_bias = to_dev(tensor)
            elif rest == "mlp.c_proj.weight":
                lw.w_down = to_dev(tensor.t().contiguous())  # [H, I]
            elif rest == "mlp.c_proj.bias":
                lw.w_down_bias = to_dev(tensor)
        if hi == s.n_layers and self.lm_head is None and self.embed is not None:
            self.lm_head = self.embed  # tied
        return self



    # ------------------------------------------------------- hybrid stacks

    @torch.no_grad()
    def _load_nukopel(self, model_path: str) -> "ModelWeights":
        """Nukopel safetensors: 'embed', 'head', 'final.norm', and per layer
        'l<i>.norm1|norm1b|norm2|norm2b' (scalars), 'l<i>.canon1',
        'l<i>.mix.*', 'l<i>.mlp.router|e<k>.*|shared.*'. All linear weights
        are [out, in]."""
        tensors = dict(iter_safetensors(model_path))
        self._assemble_hybrid(lambda name: tensors.pop(name))
        return self

    @torch.no_grad()
    def _random_init_hybrid(self, seed: int) -> "ModelWeights":
        """Random weights under the checkpoint's tensor names, assembled by
        the same code as a loaded checkpoint."""
        import zlib

        s = self.spec
        W = s.hidden_size

        def get(name: str) -> torch.Tensor:
            tseed = (seed * 1000003 + zlib.crc32(name.encode())) % (2**31)
            gen = torch.Generator(device=self.device).manual_seed(tseed)
            shape, std = self._hybrid_shape(name)
            t = torch.randn(tuple(shape), generator=gen, dtype=torch.float32,
                            device=self.device)
            if std is None:               # gains / norm weights: around 1
                return (1.0 + 0.1 * t).bfloat16()
            return (t * std).bfloat16()

        self._assemble_hybrid(get)
        return self

    def _hybrid_shape(self, name: str):
        """(shape, init std or None for a gain) of a checkpoint tensor."""
        s = self.spec
        W, V = s.hidden_size, s.vocab_size
        if name == "embed":
            return (V, W), 1.0 / max(1.0, s.embed_scale)
        if name == "head":
            return (V, W), W ** -0.5
        if name == "final.norm":
            return (), None
        parts = name.split(".")
        l = s.layer_specs[int(parts[0][1:])]
        m, f, rest = l.mixer, l.ffn, ".".join(parts[1:])
        if rest in ("norm1", "norm1b", "norm2", "norm2b"):
            return (), None
        if rest == "canon1":
            return (W, s.canon_taps), 0.2
        if rest == "mix.o":
            return (W, m.heads * m.vdim), (m.heads * m.vdim) ** -0.5
        if rest == "mix.g":
            rows = m.heads if m.kind == "latent_attention" else m.heads * m.vdim
            return (rows, W), W ** -0.5
        if m.kind == "latent_attention":
            table = {"mix.q": ((m.q_size, W), W ** -0.5),
                     "mix.dkv": ((m.cache_dim, W), W ** -0.5),
                     "mix.dkv.norm": ((m.kv_rank,), None),
                     "mix.uk": ((m.heads * m.dim, m.kv_rank), m.kv_rank ** -0.5),
                     "mix.uv": ((m.heads * m.vdim, m.kv_rank), m.kv_rank ** -0.5)}
        else:
            table = {"mix.q": ((m.heads * m.dim, W), W ** -0.5),
                     "mix.k": ((m.heads * m.dim, W), W ** -0.5),
                     "mix.v": ((m.heads * m.vdim, W), W ** -0.5),
                     "mix.norm": ((m.heads * m.vdim,), None)}
        if rest in table:
            return table[rest]
        if rest == "mlp.router":
            return (f.n_experts, W), W ** -0.5
        ff = f.shared_ff if parts[2] == "shared" else f.ff
        if parts[-1] == "down":
            return (W, ff), ff ** -0.5
        return (ff, W), W ** -0.5

    def _assemble_hybrid(self, get) -> None:
        """Build the engine layout from checkpoint-named tensors:
        one fused input projection per mixer, per-head up-projection
        stacks for the latent attention, stacked expert matrices."""
        s = self.spec
        dev, dt = self.device, self.dtype

        def act(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, dt).contiguous()

        def f32(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, torch.float32).contiguous()

        def scalar(t: torch.Tensor) -> float:
            return float(t.float().reshape(()))

        self.embed = act(get("embed"))
        self.lm_head = act(get("head"))
        self.final_gain = scalar(get("final.norm"))
        for i, l in enumerate(s.layer_specs):
            lw, p, m, f = self.layers[i], f"l{i}.", l.mixer, l.ffn
            lw.gains = tuple(
                scalar(get(p + n))
                if (f is not None or n in ("norm1", "norm1b")) else 1.0
                for n in ("norm1", "norm1b", "norm2", "norm2b"))
            if s.canon_taps:
                # checkpoint [width, taps] -> tap-major [taps, width]
                lw.canon = f32(get(p + "canon1").t())
            if m.kind == "latent_attention":
                # fused input projection rows: [q | latent+rot key | gate]
                lw.wqkv = act(torch.cat([get(p + "mix.q"), get(p + "mix.dkv"),
                                         get(p + "mix.g")], dim=0))
                lw.kv_norm = f32(get(p + "mix.dkv.norm"))
                lw.w_uk = act(get(p + "mix.uk").reshape(
                    m.heads, m.dim, m.kv_rank))
                lw.w_uv = act(get(p + "mix.uv").reshape(
                    m.heads, m.vdim, m.kv_rank).transpose(1, 2))
            else:
                # fused input projection rows: [q | k | v | gate]
                lw.wqkv = act(torch.cat([get(p + "mix.q"), get(p + "mix.k"),
                                         get(p + "mix.v"), get(p + "mix.g")],
                                        dim=0))
                lw.out_norm = f32(get(p + "mix.norm"))
                lw.decay = torch.tensor(m.decay, dtype=torch.float32,
                                        device=dev)
            lw.wo = act(get(p + "mix.o"))
            if f is None:
                continue
            lw.moe_gate = f32(get(p + "mlp.router"))
            lw.moe_w_gate_up = act(torch.stack([
                torch.cat([get(f"{p}mlp.e{e}.gate"), get(f"{p}mlp.e{e}.up")],
                          dim=0) for e in range(f.n_experts)]))
            lw.moe_w_down = act(torch.stack([
                get(f"{p}mlp.e{e}.down") for e in range(f.n_experts)]))
            if f.shared_ff:
                lw.w_gate_up = act(torch.cat(
                    [get(p + "mlp.shared.gate"), get(p + "mlp.shared.up")],
                    dim=0))
                lw.w_down = act(get(p + "mlp.shared.down"))



    # ------------------------------------- weighted-sandwich (looped) stacks

    @torch.no_grad()
    def _load_pimodra(self, model_path: str) -> "ModelWeights":
        """Pimodra safetensors: 'embed' (also the output matrix),
        'final.norm', 'loop.step' [passes, width] when a block repeats, and
        per checkpoint layer 'l<i>.norm1|norm1b|norm2|norm2b' [width],
        'l<i>.mix.q|k|v|g|o|talk', 'l<i>.mlp.up|down|act' (dense) or
        'l<i>.mlp.router|e<k>.gate|up|down' (experts). Linear weights
        [out, in]."""
        tensors = dict(iter_safetensors(model_path))
        self._assemble_pimodra(lambda name: tensors.pop(name))
        return self

    @torch.no_grad()
    def _random_init_pimodra(self, seed: int) -> "ModelWeights":
        import zlib

        def get(name: str) -> torch.Tensor:
            tseed = (seed * 1000003 + zlib.crc32(name.encode())) % (2**31)
            gen = torch.Generator(device=self.device).manual_seed(tseed)
            shape, mean, std = self._pimodra_shape(name)
            t = torch.randn(tuple(shape), generator=gen, dtype=torch.float32,
                            device=self.device)
            if name.endswith("mix.talk"):
                # near the identity: a head keeps most of its own weights
                t = torch.eye(shape[0], device=self.device) / std + t
            return (mean + std * t).bfloat16()

        self._assemble_pimodra(get)
        return self

    def _pimodra_shape(self, name: str):
        """(shape, init mean, init std) of a checkpoint tensor."""
        s = self.spec
        W, V = s.hidden_size, s.vocab_size
        if name == "embed":
            return (V, W), 0.0, 1.0
        if name == "final.norm":
            return (W,), 1.0, 0.1
        if name == "loop.step":
            return (s.step_rows, W), 0.0, 0.5
        head, rest = name.split(".", 1)
        l = next(x for x in s.layer_specs if x.src == int(head[1:]))
        m, f = l.mixer, l.ffn
        lin = W ** -0.5
        if rest in ("norm1", "norm1b", "norm2", "norm2b"):
            return (W,), 1.0, 0.1
        sizes = dict(m.in_sizes)
        if rest in ("mix.q", "mix.k", "mix.v", "mix.g"):
            return (sizes[rest[4:]], W), 0.0, lin
        if rest == "mix.o":
            return (W, m.out_size), 0.0, m.out_size ** -0.5
        if rest == "mix.talk":
            return (m.heads, m.heads), 0.0, 0.1
        if rest == "mlp.up":
            return (f.ff, W), 0.0, lin
        if rest == "mlp.down":
            return (W, f.ff), 0.0, f.ff ** -0.5
        if rest == "mlp.act":
            return (4,), 0.3, 0.2
        if rest == "mlp.router":
            return (f.n_experts, W), 0.0, lin
        if rest.endswith(".down"):
            return (W, f.ff), 0.0, f.ff ** -0.5
        return (f.ff, W), 0.0, lin

    def _assemble_pimodra(self, get) -> None:
        """Engine layout of a weighted-sandwich stack: one fused input
        projection per attention [q | k | v | gate], the head-mixing matrix
        and all norm weights in fp32, the dense feed-forward's up matrix in
        the single-fc slot, stacked expert matrices [E, 2ff, W] / [E, W, ff].
        A run with weights_of shares the owning run's LayerWeights."""
        s = self.spec
        dev, dt = self.device, self.dtype

        def act(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, dt).contiguous()

        def f32(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, torch.float32).contiguous()

        self.embed = act(get("embed"))
        self.lm_head = self.embed
        self.final_norm = f32(get("final.norm"))
        if s.step_rows:
            self.step_table = f32(get("loop.step"))
        for i, l in enumerate(s.layer_specs):
            if l.weights_of is not None:
                continue
            lw, p, m, f = self.layers[i], f"l{l.src}.", l.mixer, l.ffn
            norms = []
            for n_ in ("norm1", "norm1b", "norm2", "norm2b"):
                if f is None and n_ in ("norm2", "norm2b"):
                    norms.append(None)
                else:
                    norms.append(f32(get(p + n_)))
            lw.norms = tuple(norms)
            lw.wqkv = act(torch.cat([get(p + "mix.q"), get(p + "mix.k"),
                                     get(p + "mix.v"), get(p + "mix.g")],
                                    dim=0))
            lw.talk = f32(get(p + "mix.talk"))
            lw.wo = act(get(p + "mix.o"))
            if f is None:
                continue
            if getattr(f, "n_experts", 0):
                lw.moe_gate = f32(get(p + "mlp.router"))
                lw.moe_w_gate_up = act(torch.stack([
                    torch.cat([get(f"{p}mlp.e{e}.gate"),
                               get(f"{p}mlp.e{e}.up")], dim=0)
                    for e in range(f.n_experts)]))
                lw.moe_w_down = act(torch.stack([
                    get(f"{p}mlp.e{e}.down") for e in range(f.n_experts)]))
            else:
                lw.w_gate_up = act(get(p + "mlp.up"))
                lw.w_down = act(get(p + "mlp.down"))
                lw.act_coef = f32(get(p + "mlp.act"))
        for i, l in enumerate(s.layer_specs):
            if l.weights_of is not None:
                self.layers[i] = self.layers[l.weights_of]


    # --------------------------------------------- gated parallel-form stacks

    @torch.no_grad()
    def _load_zevilorn(self, model_path: str) -> "ModelWeights":
        """Zevilorn safetensors: 'embed', 'head', 'final.norm' and per
        checkpoint layer 'l<i>.norm1', 'l<i>.rg1|rg2' (+ '.b'),
        'l<i>.mix.*' ('.left.*' / '.right.*' for a parallel mixer),
        'l<i>.mlp.router|e<k>.up|down'. Linear weights [out, in]; a bias is
        the weight's name + '.b', a conv the projection's name + '.conv'."""
        tensors = dict(iter_safetensors(model_path))
        self._assemble_zevilorn(lambda name: tensors.pop(name))
        return self

    @torch.no_grad()
    def _random_init_zevilorn(self, seed: int) -> "ModelWeights":
        import zlib

        def get(name: str) -> torch.Tensor:
            tseed = (seed * 1000003 + zlib.crc32(name.encode())) % (2**31)
            gen = torch.Generator(device=self.device).manual_seed(tseed)
            shape, mean, std = self._zevilorn_shape(name)
            t = torch.randn(tuple(shape), generator=gen, dtype=torch.float32,
                            device=self.device)
            if name.endswith("mix.talk"):
                # near the identity: a head keeps most of its own scores
                t = torch.eye(shape[0], device=self.device) / std + t
            return (mean + std * t).bfloat16()

        self._assemble_zevilorn(get)
        return self

    def _zevilorn_shape(self, name: str):
        """(shape, init mean, init std) of a checkpoint tensor."""
        s = self.spec
        W, V = s.hidden_size, s.vocab_size
        lin = W ** -0.5
        if name == "embed":
            return (V, W), 0.0, 1.0
        if name == "head":
            return (V, W), 0.0, lin
        if name == "final.norm":
            return (W,), 1.0, 0.1
        head, rest = name.split(".", 1)
        l = next(x for x in s.layer_specs if x.src == int(head[1:]))
        f = l.ffn
        if rest == "norm1":
            return (W,), 1.0, 0.1
        if rest in ("rg1", "rg2"):
            return (W, W), 0.0, lin
        if rest in ("rg1.b", "rg2.b"):
            return (W,), 0.0, 0.5
        if rest == "mlp.router":
            return (f.n_experts, W), 0.0, lin
        if rest.startswith("mlp."):
            if rest.endswith(".down"):
                return (W, f.ff), 0.0, f.ff ** -0.5
            return (f.up_rows, W), 0.0, lin
        rest = rest[len("mix."):]
        m = l.mixer
        if m.kind == "parallel":
            if rest in ("left.out", "right.out"):
                return (W,), 1.0, 0.1
            side, rest = rest.split(".", 1)
            m = m.left if side == "left" else m.right
        if rest == "o":
            return (W, m.out_size), 0.0, m.out_size ** -0.5
        if rest == "o.b":
            return (W,), 0.0, 0.1
        sizes = dict(m.in_sizes)
        if m.kind == "latent_attention":
            table = {"dq": ((m.q_rank, W), 0.0, lin),
                     "q": ((m.q_size, W), 0.0, lin),
                     "dq.norm": ((m.q_rank,), 1.0, 0.1),
                     "uq": ((m.q_size, max(1, m.q_rank)), 0.0,
                            max(1, m.q_rank) ** -0.5),
                     "dkv": ((m.cache_dim, W), 0.0, lin),
                     "dkv.norm": ((m.kv_rank,), 1.0, 0.1),
                     "uk": ((m.heads * m.dim, m.kv_rank), 0.0,
                            m.kv_rank ** -0.5),
                     "uv": ((m.heads * m.vdim, m.kv_rank), 0.0,
                            m.kv_rank ** -0.5),
                     "sink": ((m.heads,), 0.0, 1.0),
                     "g": ((m.heads, W), 0.0, lin)}
            return table[rest]
        if m.kind == "gqa_attention" and rest == "talk":
            return (m.heads, m.heads), 0.0, 0.1
        if rest.endswith(".conv"):
            return (sizes[rest[:-5]], m.taps), 0.0, 0.4
        if rest.endswith(".b"):
            return (sizes[rest[:-2]],), 0.0, 0.1
        return (sizes[rest], W), 0.0, lin

    def _assemble_zevilorn(self, get) -> None:
        """Engine layout of a gated parallel-form stack: per layer ONE
        input matrix with every projection that reads the normed h (the
        mixer's and the two residual gates; models/hybrid.py gated_layout)
        and its bias vector, output projections per mixer part, the latent
        attention's per-head up-projection stacks, stacked expert matrices
        [E, ff, W] / [E, W, ff]; norm weights, conv taps (tap-major), the
        score-mixing matrix, sinks and the router in fp32. A run with
        weights_of shares the owning run's LayerWeights."""
        from types import SimpleNamespace

        from .hybrid import gated_layout, mixer_parts

        s = self.spec
        dev, dt = self.device, self.dtype
        W = s.hidden_size

        def act(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, dt).contiguous()

        def f32(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, torch.float32).contiguous()

        self.embed = act(get("embed"))
        self.lm_head = act(get("head"))
        self.final_norm = f32(get("final.norm"))
        for i, l in enumerate(s.layer_specs):
            if l.weights_of is not None:
                continue
            lw, p = self.layers[i], f"l{l.src}."
            ins, n_in = gated_layout(l, W)
            lw.layout = (ins, n_in)
            lw.norm_w = f32(get(p + "norm1"))
            w_in = torch.zeros(n_in, W, device=dev, dtype=dt)
            b_in = torch.zeros(n_in, device=dev, dtype=dt)

            def put_in(key: str, name: str, bias: bool = False) -> None:
                off, n = ins[key]
                t = get(name)
                assert t.shape == (n, W), (name, tuple(t.shape), n)
                w_in[off : off + n] = t.to(dev, dt)
                if bias:
                    b_in[off : off + n] = get(name + ".b").to(dev, dt)

            lw.mix = {}
            for pre, m in mixer_parts(l.mixer):
                q = p + "mix." + pre
                ns = lw.mix[pre] = SimpleNamespace()
                if m.kind == "gqa_attention":
                    for n_ in ("q", "k", "v"):
                        put_in(pre + n_, q + n_, m.bias)
                    if m.head_gate:
                        put_in(pre + "g", q + "g")
                    # checkpoint [channels, taps] -> tap-major [taps, channels]
                    ns.conv_w = f32(torch.cat(
                        [get(q + "q.conv"), get(q + "k.conv"),
                         get(q + "v.conv")], dim=0).t()) if m.taps else None
                    ns.talk = f32(get(q + "talk")) if m.score_mix else None
                    ns.wo_b = act(get(q + "o.b")) if m.bias else None
                elif m.kind == "latent_attention":
                    if m.q_rank:
                        put_in(pre + "dq", q + "dq")
                        ns.q_norm = f32(get(q + "dq.norm"))
                        ns.w_uq = act(get(q + "uq"))
                    else:
                        put_in(pre + "q", q + "q")
                        ns.q_norm = ns.w_uq = None
                    put_in(pre + "dkv", q + "dkv")
                    put_in(pre + "g", q + "g")
                    ns.kv_norm = f32(get(q + "dkv.norm"))
                    ns.w_uk = act(get(q + "uk").reshape(
                        m.heads, m.dim, m.kv_rank))
                    ns.w_uv = act(get(q + "uv").reshape(
                        m.heads, m.vdim, m.kv_rank).transpose(1, 2))
                    ns.sink = f32(get(q + "sink")) if m.sink else None
                    ns.wo_b = None
                else:
                    put_in(pre + "z", q + "z", True)
                    put_in(pre + "x", q + "x", True)
                    put_in(pre + "g", q + "g")
                    ns.wo_b = None
                ns.wo = act(get(q + "o"))
                if l.mixer.kind == "parallel" and \
                        l.mixer.combine == "normed_mean":
                    ns.out_norm = f32(get(p + "mix." + pre + "out"))
            put_in("rg1", p + "rg1", True)
            f = l.ffn
            if f is not None:
                put_in("rg2", p + "rg2", True)
                lw.moe_gate = f32(get(p + "mlp.router"))
                lw.moe_w_gate_up = act(torch.stack([
                    get(f"{p}mlp.e{e}.up") for e in range(f.n_experts)]))
                lw.moe_w_down = act(torch.stack([
                    get(f"{p}mlp.e{e}.down") for e in range(f.n_experts)]))
            lw.w_in, lw.b_in = w_in, b_in
        for i, l in enumerate(s.layer_specs):
            if l.weights_of is not None:
                self.layers[i] = self.layers[l.weights_of]

    # ------------------------------------------- parallel-form hybrid stacks

    @torch.no_grad()
    def _load_pugozen(self, model_path: str) -> "ModelWeights":
        """Pugozen safetensors: 'embed', 'head', 'final.norm' and per layer
        that owns tensors 'l<i>.norm1', 'l<i>.mix.*' ('.left.*' / '.right.*'
        for a parallel mixer), 'l<i>.mlp.up|down'. Linear weights [out, in]."""
        tensors = dict(iter_safetensors(model_path))
        self._assemble_pugozen(lambda name: tensors.pop(name))
        return self

    @torch.no_grad()
    def _random_init_pugozen(self, seed: int) -> "ModelWeights":
        import zlib

        def get(name: str) -> torch.Tensor:
            tseed = (seed * 1000003 + zlib.crc32(name.encode())) % (2**31)
            gen = torch.Generator(device=self.device).manual_seed(tseed)
            shape, mean, std = self._pugozen_shape(name)
            t = torch.randn(tuple(shape), generator=gen, dtype=torch.float32,
                            device=self.device)
            return (mean + std * t).bfloat16()

        self._assemble_pugozen(get)
        return self

    def _pugozen_shape(self, name: str):
        """(shape, init mean, init std) of a checkpoint tensor."""
        s = self.spec
        W, V = s.hidden_size, s.vocab_size
        if name == "embed":
            return (V, W), 0.0, 1.0 / max(1.0, s.embed_scale)
        if name == "head":
            return (V, W), 0.0, W ** -0.5
        if name == "final.norm":
            return (W,), 1.0, 0.1
        head, rest = name.split(".", 1)
        l = s.layer_specs[int(head[1:])]
        if rest == "norm1":
            return (W,), 1.0, 0.1
        if rest == "mlp.up":
            return (l.ffn.ff, W), 0.0, W ** -0.5
        if rest == "mlp.down":
            return (W, l.ffn.ff), 0.0, l.ffn.ff ** -0.5
        rest = rest[len("mix."):]
        m = l.mixer
        if m.kind == "parallel":
            side, rest = rest.split(".", 1)
            m = m.left if side == "left" else m.right
        H, D, Dv = m.heads, m.dim, m.vdim
        lin = W ** -0.5
        if rest == "o":
            return (W, H * Dv), 0.0, (H * Dv) ** -0.5
        if m.kind == "retention":
            return {"q": ((H * D, W), 0.0, lin), "k": ((H * D, W), 0.0, lin),
                    "v": ((H * Dv, W), 0.0, lin),
                    "g": ((H * Dv, W), 0.0, lin)}[rest]
        if m.kind == "sink_attention":
            G = m.kv_heads
            return {"q": ((H * D, W), 0.0, lin), "k": ((G * D, W), 0.0, lin),
                    "q.norm": ((D,), 1.0, 0.1), "k.norm": ((D,), 1.0, 0.1),
                    "temp": ((H,), 1.0, 0.2), "sink": ((H,), 0.0, 1.0)}[rest]
        G = m.kv_heads
        table = {"q": ((G * D, W), 0.0, lin), "k": ((G * D, W), 0.0, lin),
                 "v": ((H * Dv, W), 0.0, lin),
                 "q.conv": ((G * D, m.taps), 0.0, 0.4),
                 "k.conv": ((G * D, m.taps), 0.0, 0.4),
                 "v.conv": ((H * Dv, m.taps), 0.0, 0.4),
                 "b": ((H, W), 0.0, lin), "A_log": ((H,), -1.0, 0.5),
                 "norm": ((Dv,), 1.0, 0.1)}
        if m.channel_decay:
            table.update({"a1": ((m.decay_rank, W), 0.0, lin),
                          "a2": ((H * D, m.decay_rank), 0.0,
                                 m.decay_rank ** -0.5),
                          "dt_bias": ((H * D,), 0.0, 0.5)})
        else:
            table.update({"a": ((H, W), 0.0, lin), "dt_bias": ((H,), 0.0, 0.5)})
        if m.gate_rank:
            table.update({"g1": ((m.gate_rank, W), 0.0, lin),
                          "g2": ((H * Dv, m.gate_rank), 0.0,
                                 m.gate_rank ** -0.5)})
        else:
            table["g"] = ((H * Dv, W), 0.0, lin)
        return table[rest]

    def _assemble_pugozen(self, get) -> None:
        """Engine layout of a parallel-form stack: per layer ONE input GEMM
        (every projection that reads the normed h, the feed-forward's up
        included) and ONE output GEMM (mixer output projections and the
        feed-forward's down side by side along K), segments padded to
        multiples of 8 (models/hybrid.py fused_layout). A layer with
        weights_of shares the owning layer's LayerWeights object."""
        from types import SimpleNamespace

        from .hybrid import fused_layout, mixer_parts

        s = self.spec
        dev, dt = self.device, self.dtype
        W = s.hidden_size

        def act(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, dt).contiguous()

        def f32(t: torch.Tensor) -> torch.Tensor:
            return t.to(dev, torch.float32).contiguous()

        self.embed = act(get("embed"))
        self.lm_head = act(get("head"))
        self.final_norm = f32(get("final.norm"))
        for i, l in enumerate(s.layer_specs):
            if l.weights_of is not None:
                continue
            lw, p = self.layers[i], f"l{i}."
            ins, n_in, outs, n_out = fused_layout(l)
            lw.layout = (ins, n_in, outs, n_out)
            lw.norm_w = f32(get(p + "norm1"))
            w_in = torch.zeros(n_in, W, device=dev, dtype=dt)
            w_out = torch.zeros(W, n_out, device=dev, dtype=dt)

            def put_in(key: str, t: torch.Tensor) -> None:
                off, n = ins[key]
                assert t.shape == (n, W), (key, tuple(t.shape), n)
                w_in[off : off + n] = t.to(dev, dt)

            lw.mix = {}
            for pre, m in mixer_parts(l.mixer):
                q = p + "mix." + pre
                ns = lw.mix[pre] = SimpleNamespace()
                if m.kind == "retention":
                    for n_ in ("q", "k", "v", "g"):
                        put_in(pre + n_, get(q + n_))
                    ns.decay = torch.tensor(m.decay, dtype=torch.float32,
                                            device=dev)
                elif m.kind == "sink_attention":
                    put_in(pre + "q", get(q + "q"))
                    put_in(pre + "k", get(q + "k"))
                    ns.q_norm = f32(get(q + "q.norm"))
                    ns.k_norm = f32(get(q + "k.norm"))
                    ns.temp = f32(get(q + "temp"))
                    ns.sink = f32(get(q + "sink"))
                    # score = (q . k) * scale * temp_h, folded into q
                    ns.q_mult = ns.temp * m.scale
                else:
                    put_in(pre + "qkv", torch.cat(
                        [get(q + "q"), get(q + "k"), get(q + "v")], dim=0))
                    # checkpoint [channels, taps] -> tap-major [taps, channels]
                    ns.conv_w = f32(torch.cat(
                        [get(q + "q.conv"), get(q + "k.conv"),
                         get(q + "v.conv")], dim=0).t())
                    put_in(pre + "b", get(q + "b"))
                    # decay rate exp(A_log), evaluated once in fp32
                    ns.rate = torch.exp(f32(get(q + "A_log")))
                    ns.dt_bias = f32(get(q + "dt_bias"))
                    ns.norm = f32(get(q + "norm"))
                    if m.channel_decay:
                        put_in(pre + "a", get(q + "a1"))
                        ns.a2 = act(get(q + "a2"))
                    else:
                        put_in(pre + "a", get(q + "a"))
                        ns.a2 = None
                    if m.gate_rank:
                        put_in(pre + "g", get(q + "g1"))
                        ns.g2 = act(get(q + "g2"))
                    else:
                        put_in(pre + "g", get(q + "g"))
                        ns.g2 = None
                off, n = outs[pre + "o"]
                w_out[:, off : off + n] = get(q + "o").to(dev, dt)
            if l.ffn is not None:
                put_in("up", get(p + "mlp.up"))
                off, n = outs["down"]
                w_out[:, off : off + n] = get(p + "mlp.down").to(dev, dt)
            lw.w_in, lw.w_out = w_in, w_out
        for i, l in enumerate(s.layer_specs):
            if l.weights_of is not None:
                self.layers[i] = self.layers[l.weights_of]


def pimodra_config(spec: ModelSpec) -> Dict:
    """The config.json dict of a Pimodra spec (inverse of pimodra_spec)."""
    def mixer(m):
        rot = {"base": m.rope_base, "dims": m.rope_dims}
        if m.rope_scaling:
            rot["scaling"] = dict(m.rope_scaling)
        out = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
               "vdim": m.vdim, "scale": m.scale, "rot": rot}
        if m.window:
            out["mask"] = {"size": m.window}
        return out

    def mlp(f):
        if f is None:
            return None
        if getattr(f, "n_experts", 0):
            return {"kind": "moe", "expert": {"ff": f.ff},
                    "router": {"experts": f.n_experts, "top": f.top_k,
                               "groups": {"count": f.n_groups,
                                          "keep": f.keep_groups}}}
        return {"kind": "dense", "ff": f.ff}

    by_src = {}
    for l in spec.layer_specs:
        by_src.setdefault(l.src, l)
    layers = [{"type": "attention", "mixer": mixer(by_src[i].mixer),
               "mlp": mlp(by_src[i].ffn)} for i in sorted(by_src)]
    cfg = {"architecture": "Pimodra", "vocab": spec.vocab_size,
           "width": spec.hidden_size, "max_seq_len": spec.max_seq_len,
           "norm": {"eps": spec.rms_eps, "groups": spec.norm_groups},
           "layers": layers}
    loop = (spec.source_cfg or {}).get("loop")
    if loop:
        cfg["loop"] = dict(loop)
    return cfg


def _save_pimodra(weights: "ModelWeights", out_dir: str, tensors, cpu) -> None:
    from safetensors.torch import save_file

    s = weights.spec

    def put(name: str, t: torch.Tensor) -> None:
        tensors[name] = cpu(t).to(torch.bfloat16)

    put("embed", weights.embed)
    put("final.norm", weights.final_norm)
    if weights.step_table is not None:
        put("loop.step", weights.step_table)
    for i, l in enumerate(s.layer_specs):
        if l.weights_of is not None:
            continue
        lw, p, m, f = weights.layers[i], f"l{l.src}.", l.mixer, l.ffn
        for n_, t in zip(("norm1", "norm1b", "norm2", "norm2b"), lw.norms):
            if t is not None:
                put(p + n_, t)
        off = 0
        for n_, sz in m.in_sizes:
            put(p + "mix." + n_, lw.wqkv[off : off + sz])
            off += sz
        put(p + "mix.talk", lw.talk)
        put(p + "mix.o", lw.wo)
        if f is None:
            continue
        if getattr(f, "n_experts", 0):
            put(p + "mlp.router", lw.moe_gate)
            for e in range(f.n_experts):
                put(f"{p}mlp.e{e}.gate", lw.moe_w_gate_up[e, : f.ff])
                put(f"{p}mlp.e{e}.up", lw.moe_w_gate_up[e, f.ff :])
                put(f"{p}mlp.e{e}.down", lw.moe_w_down[e])
        else:
            put(p + "mlp.up", lw.w_gate_up)
            put(p + "mlp.down", lw.w_down)
            put(p + "mlp.act", lw.act_coef)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as fh:
        json.dump(pimodra_config(s), fh, indent=1)


def zevilorn_config(spec: ModelSpec) -> Dict:
    """The config.json dict of a Zevilorn spec (inverse of zevilorn_spec):
    the layer and loop entries are kept as they were parsed."""
    src = spec.source_cfg or {}
    cfg = {"architecture": "Zevilorn", "vocab": spec.vocab_size,
           "width": spec.hidden_size, "max_seq_len": spec.max_seq_len,
           "norm": {"eps": spec.rms_eps}, "layers": src.get("layers", [])}
    if src.get("loop"):
        cfg["loop"] = dict(src["loop"])
    return cfg


def _save_zevilorn(weights: "ModelWeights", out_dir: str, tensors, cpu) -> None:
    from safetensors.torch import save_file

    from .hybrid import mixer_parts

    s = weights.spec

    def put(name: str, t: torch.Tensor) -> None:
        tensors[name] = cpu(t).to(torch.bfloat16)

    put("embed", weights.embed)
    put("head", weights.lm_head)
    put("final.norm", weights.final_norm)
    for i, l in enumerate(s.layer_specs):
        if l.weights_of is not None:
            continue
        lw, p, f = weights.layers[i], f"l{l.src}.", l.ffn
        ins, _ = lw.layout

        def rows(key: str, name: str, bias: bool = False) -> None:
            off, n = ins[key]
            put(name, lw.w_in[off : off + n])
            if bias:
                put(name + ".b", lw.b_in[off : off + n])

        put(p + "norm1", lw.norm_w)
        rows("rg1", p + "rg1", True)
        for pre, m in mixer_parts(l.mixer):
            q, ns = p + "mix." + pre, lw.mix[pre]
            if m.kind == "gqa_attention":
                off = 0
                for n_, sz in m.in_sizes:
                    rows(pre + n_, q + n_, m.bias and n_ != "g")
                    if ns.conv_w is not None and n_ != "g":
                        put(q + n_ + ".conv", ns.conv_w[:, off : off + sz].t())
                        off += sz
                if ns.talk is not None:
                    put(q + "talk", ns.talk)
                if ns.wo_b is not None:
                    put(q + "o.b", ns.wo_b)
            elif m.kind == "latent_attention":
                if m.q_rank:
                    rows(pre + "dq", q + "dq")
                    put(q + "dq.norm", ns.q_norm)
                    put(q + "uq", ns.w_uq)
                else:
                    rows(pre + "q", q + "q")
                rows(pre + "dkv", q + "dkv")
                rows(pre + "g", q + "g")
                put(q + "dkv.norm", ns.kv_norm)
                put(q + "uk", ns.w_uk.reshape(m.heads * m.dim, m.kv_rank))
                put(q + "uv", ns.w_uv.transpose(1, 2).reshape(
                    m.heads * m.vdim, m.kv_rank))
                if ns.sink is not None:
                    put(q + "sink", ns.sink)
            else:
                rows(pre + "z", q + "z", True)
                rows(pre + "x", q + "x", True)
                rows(pre + "g", q + "g")
            put(q + "o", ns.wo)
            if hasattr(ns, "out_norm"):
                put(q + "out", ns.out_norm)
        if f is not None:
            rows("rg2", p + "rg2", True)
            put(p + "mlp.router", lw.moe_gate)
            for e in range(f.n_experts):
                put(f"{p}mlp.e{e}.up", lw.moe_w_gate_up[e])
                put(f"{p}mlp.e{e}.down", lw.moe_w_down[e])
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as fh:
        json.dump(zevilorn_config(s), fh, indent=1)


def safetensors_shapes(model_path: str) -> Dict[str, Tuple[int, ...]]:
    """Tensor name -> shape from the shards' headers (8-byte little-endian
    length, then that many bytes of JSON); no tensor data is read."""
    import struct

    out: Dict[str, Tuple[int, ...]] = {}
    for shard in sorted(glob.glob(os.path.join(model_path, "*.safetensors"))):
        with open(shard, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            header = json.loads(f.read(n))
        for name, meta in header.items():
            if name != "__metadata__":
                out[name] = tuple(meta["shape"])
    return out


def pugozen_config(spec: ModelSpec) -> Dict:
    """The config.json dict of a Pugozen spec (inverse of pugozen_spec)."""
    def rot(m):
        return {"base": m.rope_base, "dims": m.rope_dims}

    def delta(m):
        return {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                "vdim": m.vdim, "conv": m.taps}

    layers = []
    for l in spec.layer_specs:
        m = l.mixer
        if m.kind == "retention":
            mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim,
                     "decay": list(m.decay), "rot": rot(m)}
        elif m.kind == "delta":
            mixer = delta(m)
        else:
            a = m.left
            mixer = {"left": {"heads": a.heads, "kv_heads": a.kv_heads,
                              "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                              "rot": rot(a)},
                     "right": delta(m.right), "left_scale": m.left_scale,
                     "right_scale": m.right_scale}
        entry = {"type": m.kind, "mixer": mixer,
                 "mlp": ({"kind": "dense", "ff": l.ffn.ff}
                         if l.ffn is not None else None)}
        if l.weights_of is not None:
            entry["weights_of"] = l.weights_of
        layers.append(entry)
    return {"architecture": "Pugozen", "vocab": spec.vocab_size,
            "width": spec.hidden_size,
            "embedding": {"scale": spec.embed_scale},
            "norm": {"eps": spec.rms_eps}, "max_seq_len": spec.max_seq_len,
            "layers": layers}


def _save_pugozen(weights: "ModelWeights", out_dir: str, tensors, cpu) -> None:
    """Pugozen-format shard + config: the two fused matrices split back
    into the checkpoint's tensors (bf16, [out, in])."""
    from safetensors.torch import save_file

    from .hybrid import mixer_parts

    s = weights.spec

    def put(name: str, t: torch.Tensor) -> None:
        tensors[name] = cpu(t).to(torch.bfloat16).contiguous()

    put("embed", weights.embed)
    put("head", weights.lm_head)
    put("final.norm", weights.final_norm)
    for i, l in enumerate(s.layer_specs):
        if l.weights_of is not None:
            continue
        lw, p = weights.layers[i], f"l{i}."
        ins, _, outs, _ = lw.layout

        def rows(key: str) -> torch.Tensor:
            off, n = ins[key]
            return lw.w_in[off : off + n]

        put(p + "norm1", lw.norm_w)
        for pre, m in mixer_parts(l.mixer):
            q, ns = p + "mix." + pre, lw.mix[pre]
            if m.kind == "retention":
                for n_ in ("q", "k", "v", "g"):
                    put(q + n_, rows(pre + n_))
            elif m.kind == "sink_attention":
                put(q + "q", rows(pre + "q"))
                put(q + "k", rows(pre + "k"))
                put(q + "q.norm", ns.q_norm)
                put(q + "k.norm", ns.k_norm)
                put(q + "temp", ns.temp)
                put(q + "sink", ns.sink)
            else:
                nq = m.kv_heads * m.dim
                parts = torch.split(rows(pre + "qkv"),
                                    [nq, nq, m.heads * m.vdim], dim=0)
                convs = torch.split(ns.conv_w.t(), [nq, nq, m.heads * m.vdim],
                                    dim=0)
                for n_, t, c in zip("qkv", parts, convs):
                    put(q + n_, t)
                    put(q + n_ + ".conv", c)
                put(q + "b", rows(pre + "b"))
                put(q + "A_log", torch.log(ns.rate))
                put(q + "dt_bias", ns.dt_bias)
                put(q + "norm", ns.norm)
                if m.channel_decay:
                    put(q + "a1", rows(pre + "a"))
                    put(q + "a2", ns.a2)
                else:
                    put(q + "a", rows(pre + "a"))
                if m.gate_rank:
                    put(q + "g1", rows(pre + "g"))
                    put(q + "g2", ns.g2)
                else:
                    put(q + "g", rows(pre + "g"))
            off, n = outs[pre + "o"]
            put(q + "o", lw.w_out[:, off : off + n])
        if l.ffn is not None:
            put(p + "mlp.up", rows("up"))
            off, n = outs["down"]
            put(p + "mlp.down", lw.w_out[:, off : off + n])
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as fh:
        json.dump(pugozen_config(s), fh, indent=1)


def _save_gpt2(weights: "ModelWeights", out_dir: str, tensors, cpu) -> None:
    """GPT-2-format shard + config (Conv1D tensors re-transposed)."""
    from safetensors.torch import save_file

    s = weights.spec
    if weights.embed is not None:
        tensors["wte.weight"] = cpu(weights.embed)
    if weights.pos_embed is not None:
        tensors["wpe.weight"] = cpu(weights.pos_embed)
    if weights.final_norm is not None:
        tensors["ln_f.weight"] = cpu(weights.final_norm)
    if weights.final_norm_bias is not None:
        tensors["ln_f.bias"] = cpu(weights.final_norm_bias)
    for i, lw in enumerate(weights.layers):
        if lw.wqkv is None:
            continue
        p = f"h.{i}"
        tensors[f"{p}.ln_1.weight"] = cpu(lw.attn_norm)
        tensors[f"{p}.ln_1.bias"] = cpu(lw.attn_norm_bias)
        tensors[f"{p}.ln_2.weight"] = cpu(lw.mlp_norm)
        tensors[f"{p}.ln_2.bias"] = cpu(lw.mlp_norm_bias)
        tensors[f"{p}.attn.c_attn.weight"] = cpu(lw.wqkv.t())
        tensors[f"{p}.attn.c_attn.bias"] = cpu(lw.wqkv_bias)
        tensors[f"{p}.attn.c_proj.weight"] = cpu(lw.wo.t())
        tensors[f"{p}.attn.c_proj.bias"] = cpu(lw.wo_bias)
        tensors[f"{p}.mlp.c_fc.weight"] = cpu(lw.w_gate_up.t())
        tensors[f"{p}.mlp.c_fc.bias"] = cpu(lw.w_gate_up_bias)
        tensors[f"{p}.mlp.c_proj.weight"] = cpu(lw.w_down.t())
        tensors[f"{p}.mlp.c_proj.bias"] = cpu(lw.w_down_bias)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    cfg = {
        "architectures": ["GPT2LMHeadModel"],
        "model_type": "gpt2",
        "vocab_size": s.vocab_size,
        "n_embd": s.hidden_size,
        "n_layer": s.n_layers,
        "n_head": s.n_heads,
        "n_positions": s.max_seq_len,
        "layer_norm_epsilon": s.rms_eps,
        "tie_word_embeddings": True,
        "bos_token_id": s.bos_token_id,
        "eos_token_id": s.eos_token_id,
    }
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)


def nukopel_config(spec: ModelSpec) -> Dict:
    """The config.json dict of a hybrid spec (inverse of nukopel_spec)."""
    layers = []
    for l in spec.layer_specs:
        m, f = l.mixer, l.ffn
        if m.kind == "latent_attention":
            mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                     "vdim": m.vdim, "kv_rank": m.kv_rank,
                     "mask": {"size": m.window},
                     "rot": {"base": m.rope_base, "dims": m.rope_dims},
                     "scale": m.scale}
        else:
            mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim,
                     "decay": list(m.decay)}
        mlp = None
        if f is not None:
            mlp = {"kind": "moe",
                   "expert": {"ff": f.ff, "limit": f.limit},
                   "router": {"experts": f.n_experts, "top": f.top_k},
                   "shared": ({"ff": f.shared_ff, "limit": f.shared_limit}
                              if f.shared_ff else None)}
        layers.append({"type": m.kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Nukopel", "vocab": spec.vocab_size,
            "width": spec.hidden_size, "canon": {"taps": spec.canon_taps},
            "embedding": {"scale": spec.embed_scale},
            "norm": {"eps": spec.rms_eps}, "max_seq_len": spec.max_seq_len,
            "layers": layers}


def _save_nukopel(weights: "ModelWeights", out_dir: str, tensors, cpu) -> None:
    """Nukopel-format shard + config: the fused/stacked engine layout split
    back into the checkpoint's tensors (bf16, [out, in])."""
    from safetensors.torch import save_file

    s = weights.spec

    def put(name: str, t: torch.Tensor) -> None:
        tensors[name] = cpu(t).to(torch.bfloat16).contiguous()

    def gain(name: str, g: float) -> None:
        tensors[name] = torch.tensor(g, dtype=torch.bfloat16)

    put("embed", weights.embed)
    put("head", weights.lm_head)
    gain("final.norm", weights.final_gain)
    for i, l in enumerate(s.layer_specs):
        lw, p, m, f = weights.layers[i], f"l{i}.", l.mixer, l.ffn
        names = ("norm1", "norm1b") + (("norm2", "norm2b") if f else ())
        for n, g in zip(names, lw.gains):
            gain(p + n, g)
        if lw.canon is not None:
            put(p + "canon1", lw.canon.t())
        H = m.heads
        if m.kind == "latent_attention":
            q, dkv, g = torch.split(
                lw.wqkv, [m.q_size, m.cache_dim, H], dim=0)
            put(p + "mix.q", q)
            put(p + "mix.dkv", dkv)
            put(p + "mix.g", g)
            put(p + "mix.dkv.norm", lw.kv_norm)
            put(p + "mix.uk", lw.w_uk.reshape(H * m.dim, m.kv_rank))
            put(p + "mix.uv", lw.w_uv.transpose(1, 2).reshape(
                H * m.vdim, m.kv_rank))
        else:
            q, k, v, g = torch.split(
                lw.wqkv, [H * m.dim, H * m.dim, H * m.vdim, H * m.vdim], dim=0)
            for n, t in (("q", q), ("k", k), ("v", v), ("g", g)):
                put(p + "mix." + n, t)
            put(p + "mix.norm", lw.out_norm)
        put(p + "mix.o", lw.wo)
        if f is None:
            continue
        put(p + "mlp.router", lw.moe_gate)
        for e in range(f.n_experts):
            ge, up = torch.split(lw.moe_w_gate_up[e], [f.ff, f.ff], dim=0)
            put(f"{p}mlp.e{e}.gate", ge)
            put(f"{p}mlp.e{e}.up", up)
            put(f"{p}mlp.e{e}.down", lw.moe_w_down[e])
        if f.shared_ff:
            ge, up = torch.split(lw.w_gate_up, [f.shared_ff, f.shared_ff], dim=0)
            put(p + "mlp.shared.gate", ge)
            put(p + "mlp.shared.up", up)
            put(p + "mlp.shared.down", lw.w_down)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as fh:
        json.dump(nukopel_config(s), fh, indent=1)


def iter_safetensors(model_path: str) -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield (name, tensor) from every *.safetensors shard in a directory."""
    from safetensors import safe_open

    shards = sorted(glob.glob(os.path.join(model_path, "*.safetensors")))
    if not shards:
        raise FileNotFoundError(f"no safetensors shards in {model_path}")
    for shard in shards:
        with safe_open(shard, framework="pt", device="cpu") as f:
            for name in f.keys():
                yield name, f.get_tensor(name)


def save_hf(weights: ModelWeights, out_dir: str) -> None:
    """Write weights back out as one HF-format safetensors shard + config
    (checkpoint compatibility round-trip; used by tests)."""
    from safetensors.torch import save_file

    s = weights.spec
    os.makedirs(out_dir, exist_ok=True)
    tensors: Dict[str, torch.Tensor] = {}

    def cpu(t: torch.Tensor) -> torch.Tensor:
        return t.detach().to("cpu").contiguous()

    if s.arch == "gpt2":
        _save_gpt2(weights, out_dir, tensors, cpu)
        return
    if s.is_hybrid:
        if s.arch == "pugozen":
            _save_pugozen(weights, out_dir, tensors, cpu)
        elif s.arch == "pimodra":
            _save_pimodra(weights, out_dir, tensors, cpu)
        elif s.arch == "zevilorn":
            _save_zevilorn(weights, out_dir, tensors, cpu)
        else:
            _save_nukopel(weights, out_dir, tensors, cpu)
        return

    if weights.embed is not None:
        tensors["model.embed_tokens.weight"] = cpu(weights.embed)
    if weights.final_norm is not None:
        tensors["model.norm.weight"] = cpu(weights.final_norm)
    if weights.lm_head is not None and not s.tie_embeddings:
        tensors["lm_head.weight"] = cpu(weights.lm_head)
    for i, lw in enumerate(weights.layers):
        if lw.wqkv is None:
            continue
        pfx = f"model.layers.{i}"
        q, k, v = torch.split(lw.wqkv, [s.q_size, s.kv_size, s.kv_size], dim=0)
        tensors[f"{pfx}.self_attn.q_proj.weight"] = cpu(q)
        tensors[f"{pfx}.self_attn.k_proj.weight"] = cpu(k)
        tensors[f"{pfx}.self_attn.v_proj.weight"] = cpu(v)
        if lw.wqkv_bias is not None:
            qb, kb, vb = torch.split(
                lw.wqkv_bias, [s.q_size, s.kv_size, s.kv_size], dim=0
            )
            tensors[f"{pfx}.self_attn.q_proj.bias"] = cpu(qb)
            tensors[f"{pfx}.self_attn.k_proj.bias"] = cpu(kb)
            tensors[f"{pfx}.self_attn.v_proj.bias"] = cpu(vb)
        tensors[f"{pfx}.self_attn.o_proj.weight"] = cpu(lw.wo)
        tensors[f"{pfx}.input_layernorm.weight"] = cpu(lw.attn_norm)
        tensors[f"{pfx}.post_attention_layernorm.weight"] = cpu(lw.mlp_norm)
        if s.is_moe:
            tensors[f"{pfx}.block_sparse_moe.gate.weight"] = cpu(lw.moe_gate)
            for e in range(s.n_experts):
                g, u = torch.split(
                    lw.moe_w_gate_up[e], [s.intermediate_size, s.intermediate_size], dim=0
                )
                tensors[f"{pfx}.block_sparse_moe.experts.{e}.w1.weight"] = cpu(g)
                tensors[f"{pfx}.block_sparse_moe.experts.{e}.w3.weight"] = cpu(u)
                tensors[f"{pfx}.block_sparse_moe.experts.{e}.w2.weight"] = cpu(
                    lw.moe_w_down[e]
                )
        else:
            g, u = torch.split(
                lw.w_gate_up, [s.intermediate_size, s.intermediate_size], dim=0
            )
            tensors[f"{pfx}.mlp.gate_proj.weight"] = cpu(g)
            tensors[f"{pfx}.mlp.up_proj.weight"] = cpu(u)
            tensors[f"{pfx}.mlp.down_proj.weight"] = cpu(lw.w_down)

    save_file(tensors, os.path.join(out_dir, "model.safetensors"))
    cfg = {
        "architectures": ["MixtralForCausalLM" if s.is_moe else "LlamaForCausalLM"],
        "vocab_size": s.vocab_size,
        "hidden_size": s.hidden_size,
        "intermediate_size": s.intermediate_size,
        "num_hidden_layers": s.n_layers,
        "num_attention_heads": s.n_heads,
        "num_key_value_heads": s.n_kv_heads,
        "head_dim": s.head_dim,
        "rope_theta": s.rope_theta,
        "attention_bias": s.qkv_bias,
        "rms_norm_eps": s.rms_eps,
        "max_position_embeddings": s.max_seq_len,
        "tie_word_embeddings": s.tie_embeddings,
        "bos_token_id": s.bos_token_id,
        "eos_token_id": s.eos_token_id,
    }
    if s.is_moe:
        cfg["num_local_experts"] = s.n_experts
        cfg["num_experts_per_tok"] = s.top_k_experts
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2)
