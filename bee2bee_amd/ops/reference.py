"""Pure-PyTorch fp32 reference implementations of every engine op.

These are the numerics ground truth that the HIP kernels are tested against
(tests/test_ops_gpu.py compares each CDNA4 kernel to these at fp32), and the
CPU execution path for GPU-less environments (plumbing tests, BASELINE
config 1). On a GPU box the engine REQUIRES the HIP extension — see
ops/__init__.py dispatch.

Conventions (shared with the HIP kernels):
  x        [T, H]            activations (T = tokens in batch/chunk)
  q        [T, n_heads, hd]
  k, v     [T, n_kv, hd]
  k_cache  [n_blocks, n_kv, block_size, hd]   paged KV pool
  block_table [B, max_blocks] int32
  slot_mapping [T] int32     flat slot = block_id * block_size + offset
  cos/sin  [max_len, hd/2]   fp32 RoPE tables (host-precomputed)
RoPE is llama-style rotate_half: pair (i, i + hd/2).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    norm = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (norm * weight.float()).to(x.dtype)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return rmsnorm(new_residual, weight, eps), new_residual


def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor,
              eps: float) -> torch.Tensor:
    xf = x.float()
    mean = xf.mean(-1, keepdim=True)
    var = xf.var(-1, unbiased=False, keepdim=True)
    out = (xf - mean) * torch.rsqrt(var + eps)
    return (out * weight.float() + bias.float()).to(x.dtype)


def fused_add_layernorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
    bias: torch.Tensor, eps: float,
) -> Tuple[torch.Tensor, torch.Tensor]:
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return layernorm(new_residual, weight, bias, eps), new_residual


def gelu(x: torch.Tensor) -> torch.Tensor:
    """HF gelu_new (tanh approximation) — GPT-2's activation."""
    xf = x.float()
    c = 0.7978845608028654 * (xf + 0.044715 * xf.pow(3))
    return (0.5 * xf * (1.0 + torch.tanh(c))).to(x.dtype)


def rope_tables(
    max_len: int, head_dim: int, theta: float, device, dtype=torch.float32,
    scaling: "Optional[dict]" = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Host-precomputed cos/sin tables. `scaling` supports the llama3
    rope_type (Llama-3.1/3.2 checkpoints): frequencies below the low-freq
    wavelength divide by `factor`, above high-freq stay, in between
    interpolate smoothly — matches transformers' llama3 rope init."""
    import math

    inv_freq = 1.0 / (
        theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim)
    )
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = float(scaling["factor"])
        lo_f = float(scaling.get("low_freq_factor", 1.0))
        hi_f = float(scaling.get("high_freq_factor", 4.0))
        orig = float(scaling.get("original_max_position_embeddings", 8192))
        low_wl = orig / lo_f
        high_wl = orig / hi_f
        wavelen = 2 * math.pi / inv_freq
        scaled = torch.where(wavelen > low_wl, inv_freq / factor, inv_freq)
        smooth = (orig / wavelen - lo_f) / (hi_f - lo_f)
        mid = (1 - smooth) * inv_freq / factor + smooth * inv_freq
        is_mid = (wavelen <= low_wl) & (wavelen >= high_wl)
        inv_freq = torch.where(is_mid, mid, scaled)
    t = torch.arange(max_len, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)  # [max_len, hd/2]
    return freqs.cos().to(device, dtype), freqs.sin().to(device, dtype)


def rope_inplace(
    q: torch.Tensor,
    k: torch.Tensor,
    positions: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
) -> None:
    hd = q.shape[-1]
    c = cos[positions].unsqueeze(1)  # [T, 1, hd/2]
    s = sin[positions].unsqueeze(1)
    for t in (q, k):
        # .float() is identity for fp32 tensors — clone so the first-half
        # write cannot alias the second-half read
        tf = t.detach().clone().float()
        x1, x2 = tf[..., : hd // 2], tf[..., hd // 2 :]
        t[..., : hd // 2] = (x1 * c - x2 * s).to(t.dtype)
        t[..., hd // 2 :] = (x2 * c + x1 * s).to(t.dtype)


def _kv_deq(cache: torch.Tensor) -> torch.Tensor:
    """Dequantize an fp8 (OCP e4m3, uint8 storage) cache to fp32; bf16/fp32
    caches pass through as fp32."""
    if cache.dtype == torch.uint8:
        return cache.view(torch.float8_e4m3fn).float()
    return cache.float()


def _kv_quant_like(x: torch.Tensor, cache: torch.Tensor) -> torch.Tensor:
    if cache.dtype == torch.uint8:
        return x.float().to(torch.float8_e4m3fn).view(torch.uint8)
    return x.to(cache.dtype)


def kv_cache_store(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    n_blocks, n_kv, block_size, hd = k_cache.shape
    blk = torch.div(slot_mapping, block_size, rounding_mode="floor").long()
    off = (slot_mapping % block_size).long()
    k_cache[blk, :, off, :] = _kv_quant_like(k, k_cache)
    v_cache[blk, :, off, :] = _kv_quant_like(v, v_cache)


def attn_decode(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
    out_ml: torch.Tensor = None,
) -> torch.Tensor:
    """Paged single-token attention, GQA. q [B, nq, hd] -> out [B, nq, hd].
    When out_ml [B, nq, 2] is given, also writes the flash merge state
    (max scaled score m, sum-exp l) per query head — the cross-rank
    exchange for context parallelism."""
    B, nq, hd = q.shape
    _nb, n_kv, block_size, _ = k_cache.shape
    group = nq // n_kv
    out = torch.empty_like(q)
    for b in range(B):
        L = int(seq_lens[b])
        if L == 0:
            # empty context (a CP rank owning no pages of this sequence):
            # zero output with (m, l) = (-inf, 0) merge state
            out[b] = 0
            if out_ml is not None:
                out_ml[b, :, 0] = -1e30
                out_ml[b, :, 1] = 0.0
            continue
        nblk = (L + block_size - 1) // block_size
        blocks = block_table[b, :nblk].long()
        keys = _kv_deq(k_cache[blocks])  # [nblk, n_kv, bs, hd]
        vals = _kv_deq(v_cache[blocks])
        keys = keys.permute(1, 0, 2, 3).reshape(n_kv, nblk * block_size, hd)[:, :L]
        vals = vals.permute(1, 0, 2, 3).reshape(n_kv, nblk * block_size, hd)[:, :L]
        qb = q[b].float().view(n_kv, group, hd)
        scores = torch.einsum("kgd,kld->kgl", qb, keys) * scale
        probs = torch.softmax(scores, dim=-1)
        ob = torch.einsum("kgl,kld->kgd", probs, vals)
        out[b] = ob.reshape(nq, hd).to(q.dtype)
        if out_ml is not None:
            m = scores.amax(dim=-1)                         # [n_kv, group]
            l = torch.exp(scores - m.unsqueeze(-1)).sum(-1)  # [n_kv, group]
            out_ml[b, :, 0] = m.reshape(nq)
            out_ml[b, :, 1] = l.reshape(nq)
    return out


def attn_prefill(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    scale: float,
    causal: bool = True,
) -> torch.Tensor:
    """Varlen full-prompt attention, GQA. q [T, nq, hd] -> [T, nq, hd]."""
    T, nq, hd = q.shape
    n_kv = k.shape[1]
    group = nq // n_kv
    out = torch.empty_like(q)
    for i in range(cu_seqlens.numel() - 1):
        s, e = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        L = e - s
        qi = q[s:e].float().view(L, n_kv, group, hd)
        ki = k[s:e].float()
        vi = v[s:e].float()
        scores = torch.einsum("qkgd,lkd->kgql", qi, ki) * scale
        if causal:
            mask = torch.triu(
                torch.ones(L, L, dtype=torch.bool, device=q.device), diagonal=1
            )
            scores.masked_fill_(mask, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        oi = torch.einsum("kgql,lkd->qkgd", probs, vi)
        out[s:e] = oi.reshape(L, nq, hd).to(q.dtype)
    return out


def attn_decode_with_history(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    query_lens: torch.Tensor,
    scale: float,
) -> torch.Tensor:
    """Chunked-prefill attention: multiple new query tokens per sequence
    attending to the full paged history (new tokens already stored in cache).

    q [T, nq, hd] packed by sequence; seq_lens = total length incl. the new
    chunk; query_lens = chunk length per sequence."""
    T, nq, hd = q.shape
    _nb, n_kv, block_size, _ = k_cache.shape
    group = nq // n_kv
    out = torch.empty_like(q)
    t0 = 0
    for b in range(query_lens.numel()):
        QL = int(query_lens[b])
        L = int(seq_lens[b])
        nblk = (L + block_size - 1) // block_size
        blocks = block_table[b, :nblk].long()
        keys = (
            _kv_deq(k_cache[blocks])
            .permute(1, 0, 2, 3).reshape(n_kv, nblk * block_size, hd)[:, :L]
        )
        vals = (
            _kv_deq(v_cache[blocks])
            .permute(1, 0, 2, 3).reshape(n_kv, nblk * block_size, hd)[:, :L]
        )
        qb = q[t0 : t0 + QL].float().view(QL, n_kv, group, hd)
        scores = torch.einsum("qkgd,kld->kgql", qb, keys) * scale
        # causal within the chunk: query j (absolute pos L-QL+j) sees keys <= pos
        qpos = torch.arange(L - QL, L, device=q.device).view(1, 1, QL, 1)
        kpos = torch.arange(L, device=q.device).view(1, 1, 1, L)
        scores.masked_fill_(kpos > qpos, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        ob = torch.einsum("kgql,kld->qkgd", probs, vals)
        out[t0 : t0 + QL] = ob.reshape(QL, nq, hd).to(q.dtype)
        t0 += QL
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    g, u = gate_up.float().chunk(2, dim=-1)
    return (torch.nn.functional.silu(g) * u).to(gate_up.dtype)


def moe_topk_gate(
    logits: torch.Tensor, top_k: int
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Softmax-after-topk gating (Mixtral). logits [T, E] ->
    (weights [T, k] fp32, indices [T, k] int32)."""
    vals, idx = torch.topk(logits.float(), top_k, dim=-1)
    weights = torch.softmax(vals, dim=-1)
    return weights, idx.to(torch.int32)


def grouped_gemm(
    x: torch.Tensor,        # [S, K] (rows sorted by expert)
    w: torch.Tensor,        # [E, N, K]
    offsets: torch.Tensor,  # [E+1] int32
) -> torch.Tensor:
    """Per-expert segment GEMM: out[offs[e]:offs[e+1]] = x_seg @ w[e].T"""
    S, K = x.shape
    E, N, _ = w.shape
    out = torch.zeros(S, N, dtype=x.dtype, device=x.device)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            out[lo:hi] = (x[lo:hi].float() @ w[e].float().t()).to(x.dtype)
    return out


def attn_decode_lse(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
):
    """attn_decode + per-head (m, l) merge state (see parallel/cp.py)."""
    out_ml = torch.empty(q.shape[0], q.shape[1], 2, dtype=torch.float32,
                         device=q.device)
    out = attn_decode(q, k_cache, v_cache, block_table, seq_lens, scale,
                      out_ml=out_ml)
    return out, out_ml


# ------------------------------------------------------------ hybrid stacks
#
# Batch conventions for the varlen ops below (one step = B sequence chunks
# packed into T rows; a decode token is a chunk of length 1):
#   cu_seqlens  [B+1] int32   row range of each chunk
#   seq_idx     [T]   int32   chunk index of each row
#   positions   [T]   int32   absolute position of each row in its sequence
#   state_slots [B]   int32   per-sequence state slot (conv / recurrent state)
# State carried between steps is never trusted at a sequence's start: rows
# whose source position is negative read zeros, and a chunk that starts at
# position 0 starts from a zero recurrent state, so slots need no clearing.


def scalar_rmsnorm(x: torch.Tensor, gain: float, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm with a single scalar gain: x / sqrt(mean(x^2) + eps) * g."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * r * gain).to(out_dtype)


def add_scalar_rmsnorm(resid: torch.Tensor, y: torch.Tensor, post_gain: float,
                       pre_gain: Optional[float], eps: float,
                       out_dtype: torch.dtype,
                       y2: Optional[torch.Tensor] = None
                       ) -> Optional[torch.Tensor]:
    """resid (fp32, updated in place) += norm(y [+ y2]) * post_gain; returns
    norm(resid) * pre_gain in out_dtype (None when pre_gain is None)."""
    if y2 is not None:
        y = y.float() + y2.float()
    resid.add_(scalar_rmsnorm(y, post_gain, eps, torch.float32))
    if pre_gain is None:
        return None
    return scalar_rmsnorm(resid, pre_gain, eps, out_dtype)


def canon_conv(h: torch.Tensor, w: torch.Tensor, state: torch.Tensor,
               state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
               seq_idx: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """h + causal per-channel conv over time. h [T, C]; w [taps, C],
    tap-major (row taps-1 multiplies the current input, row 0 the oldest);
    state [n_slots, taps-1, C] holds each sequence's last taps-1 inputs and
    is advanced in place."""
    T, C = h.shape
    K = w.shape[0] - 1
    wf = w.float()
    hf = h.float()
    out = hf * (1.0 + wf[K])
    if K == 0:
        return out.to(h.dtype)
    sidx = seq_idx.long()
    rows = torch.arange(T, device=h.device)
    local = rows - cu_seqlens.long()[sidx]
    slots = state_slots.long()[sidx]
    pos = positions.long()
    for d in range(1, K + 1):
        src_local = local - d
        in_chunk = src_local >= 0
        from_chunk = hf[(rows - d).clamp(min=0)]
        from_state = state[slots, (K + src_local).clamp(0, K - 1)].float()
        val = torch.where(in_chunk[:, None], from_chunk, from_state)
        # select, never multiply: a reused slot may hold anything
        val = torch.where((pos - d >= 0)[:, None], val, torch.zeros_like(val))
        out += wf[K - d] * val
    # advance the state: the last K inputs of each sequence after this chunk
    cu = cu_seqlens.long()
    B = cu.numel() - 1
    lens = cu[1:] - cu[:-1]
    kk = torch.arange(K, device=h.device)
    src_local = lens[:, None] - K + kk[None, :]                  # [B, K]
    in_chunk = src_local >= 0
    from_chunk = h[(cu[:-1, None] + src_local).clamp(0, T - 1)]  # [B, K, C]
    st = state_slots.long()
    from_state = state[st[:, None], (K + src_local).clamp(0, K - 1)]
    new = torch.where(in_chunk[..., None], from_chunk.to(state.dtype),
                      from_state)
    live = lens > 0
    state[st[live]] = new[live]
    return out.to(h.dtype)


def _rot_half(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
              dims: int) -> torch.Tensor:
    """Rotate the first `dims` coords of x [..., D] (pair i with i+dims/2);
    cos/sin broadcast against x[..., :dims/2]."""
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


def latent_rope_store(q_rot: torch.Tensor, kv: torch.Tensor,
                      kv_norm: torch.Tensor, eps: float, kv_rank: int,
                      rope_dims: int, positions: torch.Tensor,
                      cos: torch.Tensor, sin: torch.Tensor,
                      cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """q_rot [T, H, R] (view, rotated in place); kv [T, kv_rank + R] (view):
    cache row = [rmsnorm(kv[:kv_rank]) * kv_norm | rotate(kv[kv_rank:])].
    cache [n_blocks, block_size, kv_rank + R]."""
    p = positions.long()
    c, s = cos[p], sin[p]                                   # [T, dims/2]
    q_rot.copy_(_rot_half(q_rot.float(), c[:, None], s[:, None],
                          rope_dims).to(q_rot.dtype))
    lat = kv[:, :kv_rank].float()
    lat = lat * torch.rsqrt(lat.pow(2).mean(-1, keepdim=True) + eps) * kv_norm
    kr = _rot_half(kv[:, kv_rank:].float(), c, s, rope_dims)
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping.long()] = torch.cat([lat, kr], -1).to(cache.dtype)


def latent_attn(q_abs: torch.Tensor, q_rot: torch.Tensor, gate: torch.Tensor,
                cache: torch.Tensor, block_table: torch.Tensor,
                positions: torch.Tensor, seq_idx: torch.Tensor,
                cu_seqlens: torch.Tensor, window: int,
                scale: float,
                sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Windowed softmax attention in the latent space (one shared key/value
    row per token). q_abs [H, T, C] (queries already multiplied by the key
    up-projection), q_rot [T, H, R], gate [T, H] raw (sigmoid applied here).
    Row t at position p of sequence b sees cached positions
    max(0, p - window + 1) .. p (window 0: 0 .. p). sink fp32 [H]: exp(sink)
    joins the softmax denominator, unscaled, without a value. Returns
    [H, T, C] in q_abs.dtype."""
    H, T, C = q_abs.shape
    bs = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1])
    out = torch.zeros(H, T, C, dtype=torch.float32, device=q_abs.device)
    cu = cu_seqlens.tolist()
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        pos = positions[lo:hi].long()
        k_lo = max(0, int(pos.min()) - window + 1) if window > 0 else 0
        k_hi = int(pos.max()) + 1
        kpos = torch.arange(k_lo, k_hi, device=q_abs.device)
        rows = block_table[b].long()[kpos // bs] * bs + kpos % bs
        kv = flat[rows].float()                              # [S, C+R]
        s = torch.einsum("htc,sc->hts", q_abs[:, lo:hi].float(), kv[:, :C])
        s += torch.einsum("thr,sr->hts", q_rot[lo:hi].float(), kv[:, C:])
        s *= scale
        d = pos[:, None] - kpos[None, :]
        dead = d < 0
        if window > 0:
            dead = dead | (d >= window)
        s.masked_fill_(dead[None], float("-inf"))
        if sink is None:
            p = torch.softmax(s, dim=-1)
        else:
            sk = sink.float().view(H, 1, 1)
            m = torch.maximum(s.max(-1, keepdim=True).values, sk)
            e = torch.exp(s - m)
            p = e / (e.sum(-1, keepdim=True) + torch.exp(sk - m))
        o = torch.einsum("hts,sc->htc", p, kv[:, :C])
        out[:, lo:hi] = o * torch.sigmoid(gate[lo:hi].float()).t()[..., None]
    return out.to(q_abs.dtype)


LIGHTNING_CHUNK = 64


def lightning_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                   decay: torch.Tensor, state: torch.Tensor,
                   state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
                   positions: torch.Tensor) -> torch.Tensor:
    """Decayed linear attention over packed chunks, fp32 throughout.
    q,k [T, H, D], v [T, H, Dv] are RAW projections (silu applied here);
    state [n_slots, H, D, Dv] fp32 is read (unless the chunk starts at
    position 0) and advanced in place. Returns o [T, H * Dv] fp32 with
    S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    F = torch.nn.functional
    T, H, D = q.shape
    Dv = v.shape[-1]
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    cu = cu_seqlens.tolist()
    lam = decay.float()                                   # [H]
    log_lam = torch.log(lam)
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        slot = int(state_slots[b])
        if int(positions[lo]) == 0:
            S = torch.zeros(H, D, Dv, dtype=torch.float32, device=q.device)
        else:
            S = state[slot].clone()
        for c0 in range(lo, hi, LIGHTNING_CHUNK):
            c1 = min(hi, c0 + LIGHTNING_CHUNK)
            n = c1 - c0
            qc = F.silu(q[c0:c1].float()).transpose(0, 1)   # [H, n, D]
            kc = F.silu(k[c0:c1].float()).transpose(0, 1)
            vc = F.silu(v[c0:c1].float()).transpose(0, 1)   # [H, n, Dv]
            i = torch.arange(n, device=q.device, dtype=torch.float32)
            diff = i[:, None] - i[None, :]                  # [n, n]
            M = torch.exp(log_lam[:, None, None] * diff.clamp(min=0))
            M = M * (diff >= 0)
            a = torch.bmm(qc, kc.transpose(1, 2)) * M       # [H, n, n]
            o = torch.bmm(a, vc)
            carry = torch.exp(log_lam[:, None] * (i + 1.0))  # [H, n]
            o += torch.bmm(qc, S) * carry[..., None]
            out[c0:c1] = o.transpose(0, 1)
            tail = torch.exp(log_lam[:, None] * (n - 1.0 - i))  # [H, n]
            S = S * torch.exp(log_lam * n)[:, None, None] + torch.bmm(
                (kc * tail[..., None]).transpose(1, 2), vc)
        state[slot] = S
    return out.view(T, H * Dv)


def gated_rmsnorm(x: torch.Tensor, w: torch.Tensor, gate: torch.Tensor,
                  eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """rmsnorm(x) * w * sigmoid(gate); x fp32 [T, N], gate raw [T, N]."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * r * w.float() * torch.sigmoid(gate.float())).to(out_dtype)


def clamped_glu(gate_up: torch.Tensor, limit: float,
                alpha: float) -> torch.Tensor:
    """[..., 2I] -> [..., I]: g = min(gate, limit), u = clamp(up, +-limit),
    y = g * sigmoid(alpha * g) * (u + 1)."""
    g, u = gate_up.float().chunk(2, dim=-1)
    g = g.clamp(max=limit)
    u = u.clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gate_up.dtype)


# ---------------------------------------------- parallel-form hybrid stacks
#
# Mechanisms of stacks whose layers are x += mixer(h) + ffn(h) with
# h = unit(x) * w: weighted fp32 norms, grouped-query attention with a sink
# logit, retention (decayed linear attention on rotated q/k), the gated
# delta rule with its short convolution, per-head gated output norms.
# Several ops write into a column slice of a wider activation buffer (`out`
# is a strided [T, n] view), so one GEMM can consume all of them.


def rope_tables_f64(max_len: int, dims: int, base: float, device
                    ) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin [max_len, dims/2] of angle p * base^(-2i/dims), evaluated in
    float64 and rounded once to fp32."""
    i = torch.arange(0, dims, 2, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(base), dtype=torch.float64), -i / dims)
    ang = torch.outer(torch.arange(max_len, dtype=torch.float64), inv)
    return (ang.cos().to(device, torch.float32),
            ang.sin().to(device, torch.float32))


def rmsnorm_f32(x: torch.Tensor, w: torch.Tensor, eps: float,
                out_dtype: torch.dtype) -> torch.Tensor:
    """fp32 rows -> unit(x) * w in out_dtype."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * r * w.float()).to(out_dtype)


def add_rmsnorm_f32(resid: torch.Tensor, y: torch.Tensor,
                    w: Optional[torch.Tensor], eps: float,
                    out_dtype: torch.dtype) -> Optional[torch.Tensor]:
    """resid (fp32, in place) += y; returns unit(resid) * w (None if w is)."""
    resid.add_(y.float())
    if w is None:
        return None
    return rmsnorm_f32(resid, w, eps, out_dtype)


def relu2(x: torch.Tensor, out: torch.Tensor) -> None:
    """out <- relu(x)^2 (both may be strided column slices)."""
    z = torch.relu(x.float())
    out.copy_((z * z).to(out.dtype))


def qk_norm_rope_store(q: torch.Tensor, k: torch.Tensor, q_norm: torch.Tensor,
                       k_norm: torch.Tensor, eps: float, rope_dims: int,
                       positions: torch.Tensor, cos, sin,
                       q_mult: torch.Tensor, k_cache: torch.Tensor,
                       v_cache: torch.Tensor,
                       slot_mapping: torch.Tensor) -> None:
    """q [T, H, D] (view, rewritten in place): rotate(unit(q) * q_norm) *
    q_mult[h]. k [T, G, D] (view, left as is): rotate(unit(k) * k_norm) goes
    to k_cache, k itself (the value) to v_cache, both
    [n_blocks, G, block, D] at slot_mapping."""
    T, G, D = k.shape
    bs = k_cache.shape[2]
    qf, kf = q.float(), k.float()
    qn = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * q_norm
    kn = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps) * k_norm
    if rope_dims:
        p = positions.long()
        c, s = cos[p][:, None], sin[p][:, None]
        qn = _rot_half(qn, c, s, rope_dims)
        kn = _rot_half(kn, c, s, rope_dims)
    q.copy_((qn * q_mult.float()[None, :, None]).to(q.dtype))
    slot = slot_mapping.long()
    blk, off = slot // bs, slot % bs
    k_cache[blk, :, off] = kn.to(k_cache.dtype)
    v_cache[blk, :, off] = k.to(v_cache.dtype)


def sink_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              block_table: torch.Tensor, positions: torch.Tensor,
              seq_idx: torch.Tensor, cu_seqlens: torch.Tensor,
              sink: Optional[torch.Tensor], window: int, out: torch.Tensor,
              out_scale: float) -> None:
    """Causal grouped-query attention over the pages; scores are q . k (all
    multipliers are already in q). Row t at position p of chunk b sees
    cached positions j <= p (and j > p - window when window > 0). The
    softmax denominator also holds exp(sink[h]) when sink is given.
    out [T, H * Dv] (strided view) <- attention * out_scale."""
    T, H, D = q.shape
    G, bs, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    rep = H // G
    cu = cu_seqlens.tolist()
    res = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        pos = positions[lo:hi].long()
        k_lo = max(0, int(pos.min()) - window + 1) if window > 0 else 0
        k_hi = int(pos.max()) + 1
        kpos = torch.arange(k_lo, k_hi, device=q.device)
        blk = block_table[b].long()[kpos // bs]
        keys = k_cache[blk, :, kpos % bs].float()          # [S, G, D]
        vals = v_cache[blk, :, kpos % bs].float()          # [S, G, Dv]
        qb = q[lo:hi].float().view(hi - lo, G, rep, D)
        s = torch.einsum("tgrd,sgd->grts", qb, keys)
        d = pos[:, None] - kpos[None, :]
        dead = d < 0
        if window > 0:
            dead = dead | (d >= window)
        s.masked_fill_(dead[None, None], float("-inf"))
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            sk = sink.float().view(G, rep, 1, 1)
            m = torch.maximum(m, sk)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sk - m)
        o = torch.einsum("grts,sgv->tgrv", e / den, vals)
        res[lo:hi] = o.reshape(hi - lo, H, Dv)
    out.copy_((res.view(T, H * Dv) * out_scale).to(out.dtype))


def short_conv(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor,
               state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
               seq_idx: torch.Tensor, positions: torch.Tensor,
               silu: bool = True) -> torch.Tensor:
    """Causal per-channel conv over time (+ silu) -> fp32 [T, C]. x [T, C]
    may be a strided column slice; w [taps, C] tap-major (last row is the
    current token's); state [n_slots, taps-1, C] holds each sequence's last
    taps-1 inputs and is advanced in place. Rows before position 0 are zero
    by select."""
    T, C = x.shape
    K = w.shape[0] - 1
    wf, xf = w.float(), x.float()
    out = xf * wf[K]
    if K > 0:
        sidx = seq_idx.long()
        rows = torch.arange(T, device=x.device)
        cu = cu_seqlens.long()
        local = rows - cu[sidx]
        slots = state_slots.long()[sidx]
        pos = positions.long()
        for d in range(1, K + 1):
            src = local - d
            val = torch.where((src >= 0)[:, None], xf[(rows - d).clamp(min=0)],
                              state[slots, (K + src).clamp(0, K - 1)].float())
            val = torch.where((pos - d >= 0)[:, None], val,
                              torch.zeros_like(val))
            out += wf[K - d] * val
        lens = cu[1:] - cu[:-1]
        kk = torch.arange(K, device=x.device)
        src = lens[:, None] - K + kk[None, :]                    # [B, K]
        st = state_slots.long()
        new = torch.where(
            (src >= 0)[..., None],
            x[(cu[:-1, None] + src).clamp(0, T - 1)].to(state.dtype),
            state[st[:, None], (K + src).clamp(0, K - 1)])
        live = lens > 0
        state[st[live]] = new[live]
    if silu:
        out = torch.nn.functional.silu(out)
    return out


def delta_gates(qk: torch.Tensor, n_qk_heads: int, dim: int, b: torch.Tensor,
                a: torch.Tensor, dt_bias: torch.Tensor, rate: torch.Tensor,
                channel_decay: bool):
    """The fp32 inputs of a delta-rule recurrence besides v.
    qk fp32 [T, >= 2*n_qk_heads*dim] (conv output; q heads then k heads):
    made unit vectors per head IN PLACE, x / sqrt(sum x^2 + 1e-6), q also
    times dim^-1/2. Returns beta = sigmoid(b) [T, H] and the decay
    g = exp(-rate_h * softplus(a + dt_bias)), [T, H] or (channel_decay)
    [T, H * dim]."""
    T = qk.shape[0]
    n = n_qk_heads * dim
    for j, mult in ((0, dim ** -0.5), (1, 1.0)):
        part = qk[:, j * n : (j + 1) * n].view(T, n_qk_heads, dim)
        part.mul_(torch.rsqrt(part.pow(2).sum(-1, keepdim=True) + 1e-6) * mult)
    beta = torch.sigmoid(b.float())
    sp = torch.nn.functional.softplus(a.float() + dt_bias.float())
    H = rate.numel()
    if channel_decay:
        g = torch.exp(-rate.float().view(1, H, 1) * sp.view(T, H, dim))
        g = g.reshape(T, H * dim)
    else:
        g = torch.exp(-rate.float() * sp)
    return beta.contiguous(), g.contiguous()


def delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
               beta: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
               state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
               positions: torch.Tensor) -> torch.Tensor:
    """Gated delta rule, fp32, token by token per sequence chunk.
    q, k [T, G, D] and v [T, H, Dv] fp32 (strided views allowed; value head
    h uses q/k head h // (H/G)); beta [T, H]; g [T, H] or [T, H*D] (fade of
    the memory rows that belong to key channels); state [n_slots, H, D, Dv]
    fp32 (the memory M), read unless the chunk starts at position 0,
    advanced in place. Per token, in this order:
      M <- g * M;  delta = beta (v - M^T k);  M <- M + k delta^T;  y = M^T q
    Returns y fp32 [T, H, Dv]."""
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    rep = H // G
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    per_channel = g.shape[1] != H
    cu = cu_seqlens.tolist()
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        slot = int(state_slots[b])
        if int(positions[lo]) == 0:
            S = torch.zeros(H, D, Dv, dtype=torch.float32, device=q.device)
        else:
            S = state[slot].clone()
        qq = q[lo:hi].float().repeat_interleave(rep, dim=1)
        kk = k[lo:hi].float().repeat_interleave(rep, dim=1)
        vv = v[lo:hi].float()
        gg = g[lo:hi].view(hi - lo, H, D, 1) if per_channel \
            else g[lo:hi].view(hi - lo, H, 1, 1)
        bb = beta[lo:hi]
        for t in range(hi - lo):
            S = S * gg[t]
            u = bb[t][:, None] * (vv[t] - torch.einsum("hdv,hd->hv", S, kk[t]))
            S = S + kk[t][:, :, None] * u[:, None, :]
            out[lo + t] = torch.einsum("hdv,hd->hv", S, qq[t])
        state[slot] = S
    return out


def head_gated_norm(o: torch.Tensor, w: Optional[torch.Tensor],
                    gate: torch.Tensor, gate_act: str, eps: float,
                    out: torch.Tensor, out_scale: float) -> None:
    """o fp32 [T, H, Dv]: per head unit(o) [* w (Dv, shared by heads)] *
    act(gate) * out_scale -> out [T, H*Dv] (strided view, activation dtype).
    gate [T, H*Dv] raw (strided view); act is "silu" or "sigmoid"."""
    T, H, Dv = o.shape
    of = o.float()
    y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        y = y * w.float()
    gf = gate.float().view(T, H, Dv)
    ga = torch.sigmoid(gf) if gate_act == "sigmoid" else \
        torch.nn.functional.silu(gf)
    out.copy_((y * ga * out_scale).reshape(T, H * Dv).to(out.dtype))


def retention_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                   decay: torch.Tensor, rope_dims: int, cos, sin,
                   k_scale: float, state: torch.Tensor,
                   state_slots: torch.Tensor, cu_seqlens: torch.Tensor,
                   positions: torch.Tensor) -> torch.Tensor:
    """Decayed linear attention on rotated queries/keys, fp32 throughout:
    q, k [T, H, D] raw projections are rotated by position (first rope_dims
    coordinates, pairs (i, i + rope_dims/2)), k times k_scale; per token
    M <- lam_h M + k v^T, y = M^T q. Chunked evaluation (intra-chunk decay
    matrix + carried state). Returns y fp32 [T, H*Dv]."""
    T, H, D = q.shape
    Dv = v.shape[-1]
    qf, kf = q.float(), k.float()
    if rope_dims:
        p = positions.long()
        c, s = cos[p][:, None], sin[p][:, None]
        qf = _rot_half(qf, c, s, rope_dims)
        kf = _rot_half(kf, c, s, rope_dims)
    kf = kf * k_scale
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    cu = cu_seqlens.tolist()
    log_lam = torch.log(decay.float())
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        slot = int(state_slots[b])
        if int(positions[lo]) == 0:
            S = torch.zeros(H, D, Dv, dtype=torch.float32, device=q.device)
        else:
            S = state[slot].clone()
        for c0 in range(lo, hi, LIGHTNING_CHUNK):
            c1 = min(hi, c0 + LIGHTNING_CHUNK)
            n = c1 - c0
            qc = qf[c0:c1].transpose(0, 1)                  # [H, n, D]
            kc = kf[c0:c1].transpose(0, 1)
            vc = v[c0:c1].float().transpose(0, 1)           # [H, n, Dv]
            i = torch.arange(n, device=q.device, dtype=torch.float32)
            diff = i[:, None] - i[None, :]
            M = torch.exp(log_lam[:, None, None] * diff.clamp(min=0))
            M = M * (diff >= 0)
            o = torch.bmm(torch.bmm(qc, kc.transpose(1, 2)) * M, vc)
            carry = torch.exp(log_lam[:, None] * (i + 1.0))
            o += torch.bmm(qc, S) * carry[..., None]
            out[c0:c1] = o.transpose(0, 1)
            tail = torch.exp(log_lam[:, None] * (n - 1.0 - i))
            S = S * torch.exp(log_lam * n)[:, None, None] + torch.bmm(
                (kc * tail[..., None]).transpose(1, 2), vc)
        state[slot] = S
    return out.view(T, H * Dv)


# --------------------------------------------- weighted-sandwich stacks
#
# Mechanisms of stacks whose sublayers are x += norm_b(f(norm_a(x))) with
# weighted RMS norms over equal parts of a row: the grouped norm fused with
# the fp32 residual update, rotation tables with wavelength-dependent
# frequency scaling, "rotate, then unit-norm" query/key preparation with the
# page store, windowed attention whose softmax weights are mixed across
# heads, the PolyNorm activation, the plain gated-linear-unit, and
# group-limited expert choice.


def group_rmsnorm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """fp32 rows [T, W] -> each of `groups` equal consecutive parts divided
    by its own sqrt(mean^2 + eps), the row times w; out_dtype."""
    T, W = x.shape
    xf = x.float().view(T, groups, W // groups)
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return ((xf * r).view(T, W) * w.float()).to(out_dtype)


def add_group_rmsnorm(resid: torch.Tensor, y: Optional[torch.Tensor],
                      w_post: Optional[torch.Tensor],
                      step: Optional[torch.Tensor],
                      w_pre: Optional[torch.Tensor], groups: int, eps: float,
                      out_dtype: torch.dtype) -> Optional[torch.Tensor]:
    """resid (fp32, in place) += group_norm(y) * w_post   (when y is given)
    resid += step                                      (when step is given)
    returns group_norm(resid) * w_pre                  (None if w_pre is)."""
    if y is not None:
        resid.add_(group_rmsnorm(y, w_post, groups, eps, torch.float32))
    if step is not None:
        resid.add_(step.float())
    if w_pre is None:
        return None
    return group_rmsnorm(resid, w_pre, groups, eps, out_dtype)


def rope_tables_scaled(max_len: int, dims: int, base: float,
                       scaling: Optional[dict], device
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin [max_len, dims/2], float64 angles rounded once to fp32.
    Pair i turns at f_i = base^(-2i/dims). scaling {factor, original, fast,
    slow}: with n(t) = dims ln(original / (2 pi t)) / (2 ln base), lo =
    max(floor(n(fast)), 0), hi = min(ceil(n(slow)), dims - 1) and ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the pair turns at
    f_i / factor * ramp_i + f_i (1 - ramp_i), and cos and sin carry the
    factor 0.1 ln(factor) + 1."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                    -2.0 * i / dims)
    mag = 1.0
    if scaling:
        factor = float(scaling["factor"])

        def n_of(turns: float) -> float:
            return dims * math.log(float(scaling["original"]) /
                                   (2.0 * math.pi * turns)) / (
                                       2.0 * math.log(float(base)))

        lo = max(math.floor(n_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(n_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        inv = inv / factor * ramp + inv * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = torch.outer(torch.arange(max_len, dtype=torch.float64), inv)
    return ((ang.cos() * mag).to(device, torch.float32),
            (ang.sin() * mag).to(device, torch.float32))


def rope_unit_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                    eps: float, rope_dims: int, positions: torch.Tensor,
                    cos, sin, q_mult: float, k_cache: torch.Tensor,
                    v_cache: torch.Tensor,
                    slot_mapping: torch.Tensor) -> None:
    """q [T, H, D] (view, rewritten in place): unit(rotate(q)) * q_mult.
    k [T, G, D], v [T, G, Dv] (views, left as they are): unit(rotate(k))
    goes to k_cache [n_blocks, G, block, D], v to v_cache
    [n_blocks, G, block, Dv], at slot_mapping. unit = x / sqrt(mean(x^2) +
    eps) per head, no weight, AFTER the rotation."""
    bs = k_cache.shape[2]
    qf, kf = q.float(), k.float()
    if rope_dims:
        p = positions.long()
        c, s = cos[p][:, None], sin[p][:, None]
        qf = _rot_half(qf, c, s, rope_dims)
        kf = _rot_half(kf, c, s, rope_dims)
    qf = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * q_mult
    kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps)
    q.copy_(qf.to(q.dtype))
    slot = slot_mapping.long()
    blk, off = slot // bs, slot % bs
    k_cache[blk, :, off] = kf.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)


def talk_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              block_table: torch.Tensor, positions: torch.Tensor,
              seq_idx: torch.Tensor, cu_seqlens: torch.Tensor,
              talk: torch.Tensor, gate: torch.Tensor, window: int,
              out: torch.Tensor) -> None:
    """Grouped-query attention over the pages whose softmax weights are
    mixed across heads: scores q . k (every multiplier is already in q), row
    t at position p of chunk b sees cached positions j <= p (j > p - window
    when window > 0), w_g = softmax per head, w'_h = sum_g talk[h, g] w_g,
    o_h = w'_h applied to the values of head h's own key/value head.
    out [T, H * Dv] (strided view) <- o * sigmoid(gate) (gate raw,
    [T, H * Dv], strided view)."""
    T, H, D = q.shape
    G, bs, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    rep = H // G
    cu = cu_seqlens.tolist()
    res = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    tk = talk.float()
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        pos = positions[lo:hi].long()
        k_lo = max(0, int(pos.min()) - window + 1) if window > 0 else 0
        k_hi = int(pos.max()) + 1
        kpos = torch.arange(k_lo, k_hi, device=q.device)
        blk = block_table[b].long()[kpos // bs]
        keys = k_cache[blk, :, kpos % bs].float()          # [S, G, D]
        vals = v_cache[blk, :, kpos % bs].float()          # [S, G, Dv]
        qb = q[lo:hi].float().view(hi - lo, G, rep, D)
        s = torch.einsum("tgrd,sgd->grts", qb, keys)
        d = pos[:, None] - kpos[None, :]
        dead = d < 0
        if window > 0:
            dead = dead | (d >= window)
        s.masked_fill_(dead[None, None], float("-inf"))
        w = torch.softmax(s, dim=-1).reshape(H, hi - lo, -1)   # [H, t, S]
        w = torch.einsum("hg,gts->hts", tk, w).view(G, rep, hi - lo, -1)
        o = torch.einsum("grts,sgv->tgrv", w, vals)
        res[lo:hi] = o.reshape(hi - lo, H, Dv)
    g = torch.sigmoid(gate.float())
    out.copy_((res.view(T, H * Dv) * g).to(out.dtype))


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float,
             out_dtype: torch.dtype) -> torch.Tensor:
    """[T, N] -> a unit(z) + b unit(z^2) + c unit(z^3) + e, (a, b, c, e) =
    coef, powers element by element, unit over the row; fp32 inside."""
    zf = z.float()
    c = coef.float()

    def unit(x):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)

    z2 = zf * zf
    y = c[0] * unit(zf) + c[1] * unit(z2) + c[2] * unit(z2 * zf) + c[3]
    return y.to(out_dtype)


def silu_glu(gate_up: torch.Tensor) -> torch.Tensor:
    """[..., 2I] -> [..., I]: silu(gate) * up."""
    g, u = gate_up.float().chunk(2, dim=-1)
    return (torch.nn.functional.silu(g) * u).to(gate_up.dtype)


def group_topk_gate(logits: torch.Tensor, top_k: int, n_groups: int,
                    keep_groups: int, score: str = "softmax",
                    group_top: int = 1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Group-limited choice on expert scores. logits fp32 [T, E]: scores =
    softmax over all experts (score "softmax") or the sigmoid of each logit
    ("sigmoid"); experts form n_groups equal groups of neighbours, a group's
    score is the sum of its group_top largest expert scores, experts outside
    the best keep_groups groups cannot be chosen; the top_k remaining scores
    are the weights, as they are. -> (weights [T, k] fp32, idx [T, k] int32).
    Fixed shapes and no host sync (graph-capturable)."""
    T, E = logits.shape
    if score == "sigmoid":
        s = torch.sigmoid(logits.float())
    else:
        s = torch.softmax(logits.float(), dim=-1)
    pick = s
    if n_groups > 1 and keep_groups < n_groups:
        per = s.view(T, n_groups, E // n_groups)
        if group_top <= 1:
            gs = per.max(-1).values
        else:
            gs = torch.topk(per, min(group_top, E // n_groups),
                            dim=-1).values.sum(-1)
        top_g = torch.topk(gs, keep_groups, dim=-1).indices
        allow = torch.zeros(T, n_groups, dtype=torch.bool, device=s.device)
        allow.scatter_(1, top_g, True)
        allow = allow[:, :, None].expand(T, n_groups, E // n_groups)
        pick = torch.where(allow.reshape(T, E), s, torch.full_like(s, -1.0))
    idx = torch.topk(pick, top_k, dim=-1).indices
    return s.gather(1, idx), idx.to(torch.int32)


# ------------------------------------------- gated parallel-form stacks
#
# Mechanisms of stacks whose layers are
#   x += sigmoid(g1) * mixer(h) + sigmoid(g2) * ffn(h),  h = unit(x) * w:
# the gated residual update fused with the next norm, rotation tables with a
# linear or banded frequency scaling, rotation in either pair layout with the
# page store, grouped-query attention with capped, head-mixed scores, the
# minGRU recurrence, the mean of two normed branch outputs, a norm on a
# column slice, the exact gelu.


def rope_freq_tables(max_len: int, dims: int, base: float,
                     scaling: Optional[dict], device
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin [max_len, dims/2], float64 angles rounded once to fp32. Pair
    i turns at f_i = base^(-2i/dims). scaling {"kind": "linear", factor}:
    f_i / factor. {"kind": "banded", factor, low, high, original}: with
    wavelength l = 2 pi / f_i, f_i is kept where l < original / high,
    divided by factor where l > original / low, and in between blended,
    (1 - s) f_i / factor + s f_i with s = (original / l - low) /
    (high - low)."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                    -2.0 * i / dims)
    if scaling:
        factor = float(scaling["factor"])
        if scaling.get("kind", "linear") == "linear":
            inv = inv / factor
        else:
            lo, hi = float(scaling["low"]), float(scaling["high"])
            orig = float(scaling["original"])
            wl = 2.0 * math.pi / inv
            sm = ((orig / wl - lo) / (hi - lo)) if hi != lo else \
                torch.ones_like(wl)
            blend = (1.0 - sm) * inv / factor + sm * inv
            inv = torch.where(wl < orig / hi, inv,
                              torch.where(wl > orig / lo, inv / factor, blend))
    ang = torch.outer(torch.arange(max_len, dtype=torch.float64), inv)
    return (ang.cos().to(device, torch.float32),
            ang.sin().to(device, torch.float32))


def _rot_pairs(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
               dims: int) -> torch.Tensor:
    """Rotate the first `dims` coords of x [..., D], pairing 2i with 2i+1;
    cos/sin broadcast against x[..., :dims:2]."""
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    rot = torch.stack([u * cos - v * sin, v * cos + u * sin], -1)
    return torch.cat([rot.flatten(-2), x[..., dims:]], -1)


def rope_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
               q_out: torch.Tensor, rope_dims: int, interleaved: bool,
               positions: torch.Tensor, cos, sin, q_mult: float,
               k_cache: torch.Tensor, v_cache: torch.Tensor,
               slot_mapping: torch.Tensor) -> None:
    """q [T, H, D], k [T, G, D], v [T, G, Dv] (views, any float dtype, left
    as they are unless q_out aliases q): rotate(q) * q_mult -> q_out
    [T, H, D]; rotate(k) -> k_cache [n_blocks, G, block, D]; v -> v_cache
    [n_blocks, G, block, Dv], at slot_mapping. The rotation covers the first
    rope_dims coordinates, pairs (2i, 2i+1) when interleaved, else
    (i, i + rope_dims/2)."""
    bs = k_cache.shape[2]
    qf, kf = q.float(), k.float()
    if rope_dims:
        p = positions.long()
        c, s = cos[p][:, None], sin[p][:, None]
        rot = _rot_pairs if interleaved else _rot_half
        qf, kf = rot(qf, c, s, rope_dims), rot(kf, c, s, rope_dims)
    q_out.copy_((qf * q_mult).to(q_out.dtype))
    slot = slot_mapping.long()
    blk, off = slot // bs, slot % bs
    k_cache[blk, :, off] = kf.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)


def gqa_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
             block_table: torch.Tensor, positions: torch.Tensor,
             seq_idx: torch.Tensor, cu_seqlens: torch.Tensor,
             softcap: float, talk: Optional[torch.Tensor],
             sink: Optional[torch.Tensor],
             head_gate: Optional[torch.Tensor], window: int,
             out: torch.Tensor) -> None:
    """Grouped-query attention over the pages. Scores q . k (the score
    scale is already in q); softcap > 0: s <- softcap tanh(s / softcap);
    talk fp32 [H, H]: s_h <- sum_g talk[h, g] s_g at every (row, key),
    BEFORE the softmax. Row t at position p of chunk b sees cached positions
    j <= p (j > p - window when window > 0). sink fp32 [H]: exp(sink_h)
    joins the denominator without a value. head_gate [T, H] raw (strided
    view): head h's output times sigmoid(head_gate[t, h]).
    out [T, H * Dv] (strided view)."""
    T, H, D = q.shape
    G, bs, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    rep = H // G
    cu = cu_seqlens.tolist()
    res = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        pos = positions[lo:hi].long()
        k_lo = max(0, int(pos.min()) - window + 1) if window > 0 else 0
        k_hi = int(pos.max()) + 1
        kpos = torch.arange(k_lo, k_hi, device=q.device)
        blk = block_table[b].long()[kpos // bs]
        keys = k_cache[blk, :, kpos % bs].float()          # [S, G, D]
        vals = v_cache[blk, :, kpos % bs].float()          # [S, G, Dv]
        qb = q[lo:hi].float().view(hi - lo, G, rep, D)
        s = torch.einsum("tgrd,sgd->grts", qb, keys).reshape(H, hi - lo, -1)
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if talk is not None:
            s = torch.einsum("hg,gts->hts", talk.float(), s)
        d = pos[:, None] - kpos[None, :]
        dead = d < 0
        if window > 0:
            dead = dead | (d >= window)
        s = s.masked_fill(dead[None], float("-inf"))
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            sk = sink.float().view(H, 1, 1)
            m = torch.maximum(m, sk)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sk - m)
        w = (e / den).view(G, rep, hi - lo, -1)
        o = torch.einsum("grts,sgv->tgrv", w, vals)
        res[lo:hi] = o.reshape(hi - lo, H, Dv)
    if head_gate is not None:
        res = res * torch.sigmoid(head_gate.float())[..., None]
    out.copy_(res.view(T, H * Dv).to(out.dtype))


def min_gru(z: torch.Tensor, x: torch.Tensor, g: torch.Tensor,
            state: torch.Tensor, state_slots: torch.Tensor,
            cu_seqlens: torch.Tensor, positions: torch.Tensor,
            out: torch.Tensor) -> None:
    """Element-wise gated recurrence over packed chunks, fp32 inside.
    z, x, g [T, N] raw projections (strided views): a = sigmoid(z),
    c = x + 1/2 where x >= 0 else sigmoid(x), S_t = (1 - a) S_(t-1) + a c,
    out [T, N] (strided view) <- S_t * silu(g). state [n_slots, N] fp32 is
    read unless the chunk starts at position 0 and advanced in place."""
    a = torch.sigmoid(z.float())
    xf = x.float()
    c = torch.where(xf >= 0, xf + 0.5, torch.sigmoid(xf))
    gate = torch.nn.functional.silu(g.float())
    res = torch.empty_like(xf)
    cu = cu_seqlens.tolist()
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        slot = int(state_slots[b])
        if int(positions[lo]) == 0:
            S = torch.zeros_like(xf[0])
        else:
            S = state[slot].clone()
        for t in range(lo, hi):
            S = (1.0 - a[t]) * S + a[t] * c[t]
            res[t] = S
        state[slot] = S
    out.copy_((res * gate).to(out.dtype))


def pair_rmsnorm_mean(a: torch.Tensor, wa: torch.Tensor, b: torch.Tensor,
                      wb: torch.Tensor, eps: float,
                      out_dtype: torch.dtype) -> torch.Tensor:
    """(unit(a) * wa + unit(b) * wb) / 2 over rows [T, W]."""
    def un(x):
        xf = x.float()
        return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)

    return (0.5 * (un(a) * wa.float() + un(b) * wb.float())).to(out_dtype)


def slice_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float
                  ) -> torch.Tensor:
    """unit(x) * w for rows [T, N] that may be a strided column slice;
    contiguous result in x.dtype."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * r * w.float()).to(x.dtype).contiguous()


def gated_add_rmsnorm(resid: torch.Tensor, y1: torch.Tensor,
                      g1: torch.Tensor, y2: Optional[torch.Tensor],
                      g2: Optional[torch.Tensor],
                      extra: Optional[torch.Tensor],
                      w: Optional[torch.Tensor], eps: float,
                      out_dtype: torch.dtype) -> Optional[torch.Tensor]:
    """resid (fp32, in place) += sigmoid(g1) * y1 [+ sigmoid(g2) * y2]
    [+ extra]; returns unit(resid) * w (None if w is). g1, g2 [T, W] raw
    (strided views); extra [T, W]. y1 None: only extra and the norm."""
    if y1 is not None:
        resid.add_(torch.sigmoid(g1.float()) * y1.float())
    if y2 is not None:
        resid.add_(torch.sigmoid(g2.float()) * y2.float())
    if extra is not None:
        resid.add_(extra.float())
    if w is None:
        return None
    return rmsnorm_f32(resid, w, eps, out_dtype)


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    """Exact gelu, x/2 (1 + erf(x / sqrt 2)), evaluated in fp32."""
    return torch.nn.functional.gelu(x.float()).to(x.dtype)
