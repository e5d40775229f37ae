"""Per-layer specs for hybrid decoder stacks: models whose layers differ in
mixer kind (softmax attention over a compressed latent cache, linear
attention with a decayed recurrent state) and carry their own feed-forward
sizes. A ModelSpec with `layer_specs` set is executed by the Runner's hybrid
path (engine/runner.py), cached by PagedKV's latent pages and state slots
(engine/kv.py), and its mechanisms are ops beside the dense-attention ones
(ops/__init__.py: latent_attn, lightning_attn, canon_conv, scalar norms,
clamped GLU).

Every constant a checkpoint's config.json may vary is a field here; nothing
below assumes particular sizes, head counts, window lengths or layer order.

Nukopel config.json keys (the family served through this path):
  architecture, vocab, width, canon.taps, embedding.scale, norm.eps,
  layers[i].type in {latent_attention, lightning},
  layers[i].mixer.{heads, dim, vdim, ...}, layers[i].mlp (or null).

Pugozen config.json keys (parallel-form layers: one weighted RMS norm whose
output feeds the mixer AND the feed-forward, both added to the residual):
  architecture, vocab, width, embedding.scale, norm.eps,
  layers[i].type in {retention, delta, parallel}, layers[i].weights_of,
  layers[i].mixer.{heads, kv_heads, dim, vdim, decay, conv, rot.{base,dims},
  scale, left, right, left_scale, right_scale},
  layers[i].mlp.{kind: dense, ff} (or null).

Pimodra config.json keys (weighted grouped RMS norms before and after each
sublayer; a block of layers may run several times with the same tensors):
  architecture, vocab, width, norm.{eps, groups},
  loop.{start, stop, times} (or absent),
  layers[i].type = attention,
  layers[i].mixer.{heads, kv_heads, dim, vdim, scale, mask.size,
  rot.{base, dims, scaling.{factor, original, fast, slow}}},
  layers[i].mlp.{kind: dense, ff} | {kind: moe, expert.ff,
  router.{experts, top, groups.{count, keep}}} (or null).

Zevilorn config.json keys (parallel-form layers whose two sublayer outputs
each pass a sigmoid gate computed from the normed input; a block of layers
may run several times with the same tensors, the embedding output being
added back before every later pass):
  architecture, vocab, width, norm.eps, loop.{start, stop, times} (or absent),
  layers[i].type in {attention, latent_attention, parallel},
  attention: mixer.{heads, kv_heads, dim, vdim, scale, softcap, conv,
  mask.size, rot.{base, dims, scaling.{factor, low, high, original}}},
  latent_attention: mixer.{heads, dim, rot_dim, vdim, kv_rank, q_rank, scale,
  rot.{base, dims}},
  parallel: mixer.left.{heads, kv_heads, dim, vdim, scale, mask.size,
  rot.{base, dims, scaling.{factor}}}, mixer.right.{width},
  layers[i].mlp.{kind: moe, expert.ff, router.{experts, top,
  groups.{count, keep}}} (or null).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class LatentAttnSpec:
    """Multi-head attention whose keys/values are up-projections of one
    shared low-rank latent per token. Cached per token: the normed latent
    (kv_rank) and ONE rotated key part (rot_dim) shared by all heads."""
    heads: int
    dim: int            # unrotated query/key dims per head
    rot_dim: int        # rotated query/key dims per head
    vdim: int
    kv_rank: int
    window: int         # query i sees keys j with 0 <= i - j < window;
                        # 0: every earlier position
    rope_base: float
    rope_dims: int      # leading dims of the rot part that rotate
    scale: float
    # queries through a normed latent of this width (0: one full projection)
    q_rank: int = 0
    # a learned logit per head that counts once in the softmax denominator
    # and has neither key nor value
    sink: bool = False

    kind = "latent_attention"

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        """Rows of the fused input projection, in order."""
        return (("dq" if self.q_rank else "q", self.q_rank or self.q_size),
                ("dkv", self.cache_dim), ("g", self.heads))

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim

    @property
    def q_size(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def cache_dim(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass
class LightningSpec:
    """Linear attention with a per-head scalar decay:
    S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    kind = "lightning"


@dataclass
class RetentionSpec:
    """Linear attention with a fixed per-head decay, no softmax and no
    denominator, on rotated queries/keys:
    memory M (dim x vdim per head), M <- lam_h M + (k / sqrt(dim)) v^T per
    token, read-out y = M^T q, then per-head unit norm (no weight) and a
    silu output gate."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rope_base: float = 10000.0
    rope_dims: int = 0      # leading dims of each head that rotate (0: none)

    kind = "retention"

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        """Rows of the fused input projection, in order."""
        return (("q", self.heads * self.dim), ("k", self.heads * self.dim),
                ("v", self.heads * self.vdim), ("g", self.heads * self.vdim))

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim


@dataclass
class DeltaSpec:
    """Gated delta rule with a carried fp32 memory M (dim x vdim) per
    head. Per token: fade M <- gamma * M; what the key already recalls is
    taken out of the write, delta = beta (v - M^T k); M <- M + k delta^T;
    read-out y = M^T q (it sees the token's own write).
    q/k (kv_heads x dim, shared by groups of value heads) and v pass a short
    causal per-channel convolution + silu; q, k are unit vectors.
    channel_decay: gamma is one number per head (False: projection 'a') or one
    per head and key channel (True: low-rank projection 'a2 a1').
    gate: "silu" with a full projection 'g', or "sigmoid" with the low-rank
    pair 'g2 g1'."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int
    channel_decay: bool = False
    decay_rank: int = 0
    gate: str = "silu"
    gate_rank: int = 0

    kind = "delta"

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        n_a = self.decay_rank if self.channel_decay else self.heads
        n_g = self.gate_rank if self.gate_rank else self.heads * self.vdim
        return (("qkv", self.conv_channels), ("b", self.heads), ("a", n_a),
                ("g", n_g))

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim


@dataclass
class SinkAttnSpec:
    """Causal grouped-query softmax attention over paged keys with
    per-head RMS-normed, partly rotated queries/keys, a per-head score
    multiplier and a per-head sink logit in the softmax denominator (no key,
    no value). value_from_key: the values ARE the key projection as
    projected (before norm and rotation); there is no value projection.
    window: 0 = every earlier position, else 0 <= i - j < window."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rope_base: float = 10000.0
    rope_dims: int = 0
    window: int = 0
    value_from_key: bool = True

    kind = "sink_attention"

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        return (("q", self.heads * self.dim), ("k", self.kv_heads * self.dim))

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim


@dataclass
class TalkAttnSpec:
    """Grouped-query softmax attention over paged keys and values with a
    sliding window, whose per-head softmax weights are MIXED across heads
    before they meet the values: w'_h = sum_g talk[h, g] w_g, and head h
    applies w'_h to the values of its own key/value head. Queries and keys
    are rotated (first rope_dims coordinates, pairs (i, i + rope_dims/2),
    optionally with a wavelength-dependent frequency scaling) and THEN made
    unit-RMS per head without a weight. The concatenated heads are gated by
    sigmoid of a projection of the mixer input before the output
    projection. window: 0 = every earlier position, else 0 <= i - j < window.
    rope_scaling: None or {factor, original, fast, slow}."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    rope_base: float = 10000.0
    rope_dims: int = 0
    rope_scaling: Optional[Dict[str, float]] = None

    kind = "talk_attention"

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        """Rows of the fused input projection, in order."""
        return (("q", self.heads * self.dim), ("k", self.kv_heads * self.dim),
                ("v", self.kv_heads * self.vdim),
                ("g", self.heads * self.vdim))

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim


@dataclass
class GqaAttnSpec:
    """Grouped-query softmax attention over paged keys and values whose
    extras are all options: biases on q/k/v/o, a short causal per-channel
    convolution on the projected q, k, v (taps > 1; the last taps-1
    projected rows are carried per sequence), rotation of the first
    rope_dims coordinates in the interleaved (2i, 2i+1) or half (i, i+n)
    layout with an optional frequency scaling, a tanh cap on the scaled
    scores (softcap > 0), a learned heads x heads mix of the capped scores
    BEFORE the softmax (score_mix), a sliding window (0: none), a
    zero-logit sink in the softmax denominator (zero_sink: one is added to
    the sum), and a sigmoid gate per head on the output (head_gate).
    rope_scaling: None, {"kind": "linear", "factor"} (every frequency
    divided by factor) or {"kind": "banded", "factor", "low", "high",
    "original"} (wavelengths above original/low slowed by factor, below
    original/high kept, a linear blend between)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    rope_base: float = 10000.0
    rope_dims: int = 0
    rope_layout: str = "interleaved"
    rope_scaling: Optional[Dict[str, Any]] = None
    softcap: float = 0.0
    score_mix: bool = False
    zero_sink: bool = False
    bias: bool = False
    taps: int = 0
    head_gate: bool = False

    kind = "gqa_attention"

    @property
    def conv_channels(self) -> int:
        return (self.heads + self.kv_heads) * self.dim + \
            self.kv_heads * self.vdim

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        """Rows of the fused input projection, in order (q, k, v are
        neighbours so one convolution covers them)."""
        out = (("q", self.heads * self.dim), ("k", self.kv_heads * self.dim),
               ("v", self.kv_heads * self.vdim))
        return out + ((("g", self.heads),) if self.head_gate else ())

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim


@dataclass
class MinGRUSpec:
    """Element-wise gated recurrence whose gates read only the current
    token: z = sigmoid(W_z h + b_z), u = W_x h + b_x, candidate c = u + 1/2
    (u >= 0) or sigmoid(u) (u < 0), S_t = (1 - z) S_(t-1) + z c, output
    S_t * silu(W_g h). State [width] fp32 per sequence, zero at the start."""
    width: int

    kind = "min_gru"
    heads = 1
    dim = 1

    @property
    def in_sizes(self) -> Tuple[Tuple[str, int], ...]:
        return (("z", self.width), ("x", self.width), ("g", self.width))

    @property
    def out_size(self) -> int:
        return self.width


@dataclass
class ParallelMixerSpec:
    """Two mixers on the same input. combine "scaled_sum": summed with
    fixed scales; "normed_mean": each side's projected output is RMS-normed
    over the model width with a weight of its own, then half their sum."""
    left: Any               # SinkAttnSpec | GqaAttnSpec
    right: Any              # DeltaSpec | MinGRUSpec
    left_scale: float = 1.0
    right_scale: float = 1.0
    combine: str = "scaled_sum"

    kind = "parallel"

    @property
    def heads(self) -> int:
        return max(self.left.heads, self.right.heads)

    @property
    def dim(self) -> int:
        return max(self.left.dim, self.right.dim)


@dataclass
class DenseFFNSpec:
    """down(act(up h)); act "relu2" is the square of relu; "polynorm" is
    a unit(z) + b unit(z^2) + c unit(z^3) + e with four learned numbers
    (powers element by element, unit over the ff axis)."""
    ff: int
    act: str = "relu2"


@dataclass
class MoEFFNSpec:
    """Routed experts (+ optional always-on shared expert) with the clamped
    GLU activation: g = min(gate, limit), u = clamp(up, +-limit),
    y = g * sigmoid(alpha g) * (u + 1).
    act "silu_glu": y = silu(gate) * up instead.
    score "softmax_topk": top-k on the logits, weights = softmax over the
    chosen logits. score "softmax_all": scores = softmax over ALL experts,
    the top-k scores are the weights as they are (no renormalization); with
    n_groups > 1 the experts form equal groups of neighbours, a group's
    score is its largest expert score, and only experts of the best
    keep_groups groups can be chosen. score "sigmoid_all": as "softmax_all"
    with scores = sigmoid of each logit. group_top: a group's score is the
    sum of its group_top largest expert scores.
    act "gelu": experts without a gate, y = down(gelu(up h)), exact (erf)
    gelu."""
    n_experts: int
    top_k: int
    ff: int
    limit: float = 0.0
    shared_ff: int = 0
    shared_limit: float = 0.0
    alpha: float = 1.702
    act: str = "clamped_glu"
    score: str = "softmax_topk"
    n_groups: int = 1
    keep_groups: int = 1
    group_top: int = 1

    @property
    def up_rows(self) -> int:
        """Rows of one expert's input-side matrix."""
        return self.ff if self.act == "gelu" else 2 * self.ff


@dataclass
class LayerSpec:
    mixer: Any                      # one of the mixer specs above
    ffn: Any = None                 # MoEFFNSpec | DenseFFNSpec | None
    # "sandwich": scalar-gain norms before and after each sublayer, mixer
    # then feed-forward. "parallel": x += mixer(h) + ffn(h), h = norm(x) * w.
    # "sandwich_w": as "sandwich" with weighted, grouped RMS norms.
    # "parallel_gated": x += sigmoid(W1 h + b1) * mixer(h)
    #                      + sigmoid(W2 h + b2) * ffn(h), h = norm(x) * w.
    form: str = "sandwich"
    # layer whose tensors this layer uses (its own cache and state)
    weights_of: Optional[int] = None
    # row of the model's step table added to the residual right before
    # this layer (the first layer of a pass over a repeated block)
    step_row: Optional[int] = None
    # index of the checkpoint layer ('l<src>.') this run executes
    src: Optional[int] = None
    # the embedding output is added to the residual right before this run
    # (the first layer of every pass but the first over a repeated block)
    readd_embed: bool = False

    @property
    def kind(self) -> str:
        return self.mixer.kind


def _mixer_from_cfg(kind: str, m: Dict[str, Any]):
    if kind == "latent_attention":
        rot = m.get("rot") or {}
        rot_dim = int(m["rot_dim"])
        return LatentAttnSpec(
            heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim,
            vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
            window=int(m["mask"]["size"]),
            rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", rot_dim)),
            scale=float(m["scale"]),
        )
    if kind == "lightning":
        decay = tuple(float(d) for d in m["decay"])
        if len(decay) != int(m["heads"]):
            raise ValueError("lightning mixer needs one decay per head")
        return LightningSpec(heads=int(m["heads"]), dim=int(m["dim"]),
                             vdim=int(m["vdim"]), decay=decay)
    rot = m.get("rot") or {}
    if kind == "retention":
        decay = tuple(float(d) for d in m["decay"])
        if len(decay) != int(m["heads"]):
            raise ValueError("retention mixer needs one decay per head")
        return RetentionSpec(
            heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
            decay=decay, rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", 0)))
    if kind == "delta":
        return _delta_from_cfg(m, channel_decay=False, gate="silu")
    if kind == "sink_attention":
        return SinkAttnSpec(
            heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
            dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
            scale=float(m["scale"]),
            rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", 0)))
    if kind == "parallel":
        return ParallelMixerSpec(
            left=_mixer_from_cfg("sink_attention", m["left"]),
            right=_delta_from_cfg(m["right"], channel_decay=True,
                                  gate="sigmoid"),
            left_scale=float(m["left_scale"]),
            right_scale=float(m["right_scale"]))
    raise ValueError(f"unknown mixer type {kind!r}")


def _delta_from_cfg(m: Dict[str, Any], channel_decay: bool,
                    gate: str) -> DeltaSpec:
    heads = int(m["heads"])
    kv_heads = int(m.get("kv_heads", heads))
    if heads % kv_heads:
        raise ValueError("delta mixer: heads must be a multiple of kv_heads")
    # low-rank widths are tensor shapes, not config keys: filled in by
    # complete_from_shapes() (checkpoints) or given directly (synthetic)
    return DeltaSpec(heads=heads, kv_heads=kv_heads, dim=int(m["dim"]),
                     vdim=int(m["vdim"]), taps=int(m["conv"]),
                     channel_decay=channel_decay, gate=gate,
                     decay_rank=int(m.get("decay_rank", 0)),
                     gate_rank=int(m.get("gate_rank", 0)))


def _ffn_from_cfg(f: Optional[Dict[str, Any]]) -> Optional[MoEFFNSpec]:
    if not f:
        return None
    if f.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    shared = f.get("shared") or {}
    return MoEFFNSpec(
        n_experts=int(f["router"]["experts"]), top_k=int(f["router"]["top"]),
        ff=int(f["expert"]["ff"]), limit=float(f["expert"]["limit"]),
        shared_ff=int(shared.get("ff", 0)),
        shared_limit=float(shared.get("limit", 0.0)),
    )


def layer_specs_from_cfg(layers: List[Dict[str, Any]]) -> List[LayerSpec]:
    return [LayerSpec(mixer=_mixer_from_cfg(l["type"], l["mixer"]),
                      ffn=_ffn_from_cfg(l.get("mlp"))) for l in layers]


def parallel_layer_specs_from_cfg(layers: List[Dict[str, Any]]
                                  ) -> List[LayerSpec]:
    """Parallel-form layers (Pugozen): dense feed-forward, optional
    'weights_of' (a layer that runs another layer's tensors)."""
    out = []
    for i, l in enumerate(layers):
        f = l.get("mlp")
        if f and f.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
        src = l.get("weights_of")
        if src is not None:
            # follow a chain to the layer that owns the tensors
            src, hops = int(src), 0
            while 0 <= src < len(layers) and \
                    layers[src].get("weights_of") is not None:
                src, hops = int(layers[src]["weights_of"]), hops + 1
                if hops > len(layers):
                    raise ValueError(f"layer {i}: weights_of forms a cycle")
            if not 0 <= src < len(layers) or src == i:
                raise ValueError(f"layer {i}: bad weights_of {src}")
            if layers[src]["type"] != l["type"]:
                raise ValueError(f"layer {i}: weights_of a layer of another type")
        out.append(LayerSpec(
            mixer=_mixer_from_cfg(l["type"], l["mixer"]),
            ffn=DenseFFNSpec(ff=int(f["ff"])) if f else None,
            form="parallel", weights_of=src))
    return out


def _talk_attn_from_cfg(m: Dict[str, Any]) -> TalkAttnSpec:
    heads = int(m["heads"])
    kv_heads = int(m.get("kv_heads", heads))
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    if dims % 2 or dims > int(m["dim"]):
        raise ValueError("attention: rot.dims must be even and <= dim")
    sc = rot.get("scaling") or None
    if sc is not None:
        sc = {k: float(sc[k]) for k in ("factor", "original", "fast", "slow")}
    return TalkAttnSpec(
        heads=heads, kv_heads=kv_heads, dim=int(m["dim"]),
        vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
        window=int((m.get("mask") or {}).get("size", 0) or 0),
        rope_base=float(rot.get("base", 10000.0)), rope_dims=dims,
        rope_scaling=sc)


def _pimodra_ffn_from_cfg(f: Optional[Dict[str, Any]]):
    if not f:
        return None
    kind = f.get("kind", "dense")
    if kind == "dense":
        return DenseFFNSpec(ff=int(f["ff"]), act="polynorm")
    if kind != "moe":
        raise ValueError(f"unknown feed-forward kind {kind!r}")
    r = f["router"]
    g = r.get("groups") or {}
    E, n_g = int(r["experts"]), int(g.get("count", 1))
    keep = int(g.get("keep", n_g))
    if E % n_g or not 1 <= keep <= n_g:
        raise ValueError("router: experts must split into equal groups")
    if int(r["top"]) > keep * (E // n_g):
        raise ValueError("router: top exceeds the experts of the kept groups")
    return MoEFFNSpec(n_experts=E, top_k=int(r["top"]),
                      ff=int(f["expert"]["ff"]), act="silu_glu",
                      score="softmax_all", n_groups=n_g, keep_groups=keep)


def _loop_order(n: int, loop: Optional[Dict[str, Any]]
                ) -> List[Tuple[int, Optional[int]]]:
    """[(checkpoint layer, pass number or None)] in execution order: layers
    start..stop-1 run `times` times in a row, the rest once."""
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if not (0 <= a < b <= n and times >= 1):
        raise ValueError("loop: need 0 <= start < stop <= layers, times >= 1")
    order: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def looped_layer_specs_from_cfg(layers: List[Dict[str, Any]],
                                loop: Optional[Dict[str, Any]]
                                ) -> List[LayerSpec]:
    """Pimodra: the list of layer RUNS in execution order. Layers
    start..stop-1 of the checkpoint run `times` times in a row; every run
    is a LayerSpec of its own (own pages), runs after the first pass name
    the first pass's run as `weights_of`, and the first run of each pass
    carries the pass number as `step_row`."""
    order = _loop_order(len(layers), loop)
    out: List[LayerSpec] = []
    first_run: Dict[int, int] = {}
    for run, (i, t) in enumerate(order):
        l = layers[i]
        if l["type"] != "attention":
            raise ValueError(f"unknown mixer type {l['type']!r}")
        owner = first_run.setdefault(i, run)
        out.append(LayerSpec(
            mixer=_talk_attn_from_cfg(l["mixer"]),
            ffn=_pimodra_ffn_from_cfg(l.get("mlp")), form="sandwich_w",
            weights_of=None if owner == run else owner,
            step_row=t if (t is not None and i == int(loop["start"])) else None,
            src=i))
    return out


def _rot_scaling(sc: Optional[Dict[str, Any]]) -> Optional[Dict[str, Any]]:
    """A rot.scaling entry: with 'original' the banded rule, with only a
    factor the linear one."""
    if not sc:
        return None
    if "original" in sc:
        return {"kind": "banded", "factor": float(sc["factor"]),
                "low": float(sc["low"]), "high": float(sc["high"]),
                "original": float(sc["original"])}
    return {"kind": "linear", "factor": float(sc["factor"])}


def _gqa_attn_from_cfg(m: Dict[str, Any], **options: Any) -> GqaAttnSpec:
    heads = int(m["heads"])
    kv_heads = int(m.get("kv_heads", heads))
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    if dims % 2 or dims > int(m["dim"]):
        raise ValueError("attention: rot.dims must be even and <= dim")
    return GqaAttnSpec(
        heads=heads, kv_heads=kv_heads, dim=int(m["dim"]),
        vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
        window=int((m.get("mask") or {}).get("size", 0) or 0),
        rope_base=float(rot.get("base", 10000.0)), rope_dims=dims,
        rope_layout="interleaved",
        rope_scaling=_rot_scaling(rot.get("scaling")),
        softcap=float(m.get("softcap") or 0.0),
        taps=int(m.get("conv") or 0), **options)


def _zevilorn_mixer_from_cfg(kind: str, m: Dict[str, Any]):
    if kind == "attention":
        return _gqa_attn_from_cfg(m, score_mix=True, zero_sink=True,
                                  bias=True)
    if kind == "latent_attention":
        rot = m.get("rot") or {}
        rot_dim = int(m["rot_dim"])
        dims = int(rot.get("dims", rot_dim))
        if dims % 2 or dims > rot_dim:
            raise ValueError("latent attention: rot.dims must be even and "
                             "<= rot_dim")
        return LatentAttnSpec(
            heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim,
            vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
            window=int((m.get("mask") or {}).get("size", 0) or 0),
            rope_base=float(rot.get("base", 10000.0)), rope_dims=dims,
            scale=float(m["scale"]), q_rank=int(m.get("q_rank") or 0),
            sink=True)
    if kind == "parallel":
        return ParallelMixerSpec(
            left=_gqa_attn_from_cfg(m["left"], head_gate=True),
            right=MinGRUSpec(width=int(m["right"]["width"])),
            combine="normed_mean")
    raise ValueError(f"unknown mixer type {kind!r}")


def _zevilorn_ffn_from_cfg(f: Optional[Dict[str, Any]]):
    if not f:
        return None
    if f.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    r = f["router"]
    g = r.get("groups") or {}
    E, n_g = int(r["experts"]), int(g.get("count", 1))
    keep = int(g.get("keep", n_g))
    if E % n_g or not 1 <= keep <= n_g:
        raise ValueError("router: experts must split into equal groups")
    if int(r["top"]) > keep * (E // n_g):
        raise ValueError("router: top exceeds the experts of the kept groups")
    return MoEFFNSpec(n_experts=E, top_k=int(r["top"]),
                      ff=int(f["expert"]["ff"]), act="gelu",
                      score="sigmoid_all", n_groups=n_g, keep_groups=keep,
                      group_top=min(2, E // n_g))


def gated_layer_specs_from_cfg(layers: List[Dict[str, Any]],
                               loop: Optional[Dict[str, Any]]
                               ) -> List[LayerSpec]:
    """Zevilorn: the list of layer RUNS in execution order (a repeated
    block appears once per pass; runs after the first pass name the first
    pass's run as `weights_of` and keep pages and state of their own). The
    first run of every pass but the first has `readd_embed`."""
    out: List[LayerSpec] = []
    first_run: Dict[int, int] = {}
    for run, (i, t) in enumerate(_loop_order(len(layers), loop)):
        l = layers[i]
        owner = first_run.setdefault(i, run)
        out.append(LayerSpec(
            mixer=_zevilorn_mixer_from_cfg(l["type"], l["mixer"]),
            ffn=_zevilorn_ffn_from_cfg(l.get("mlp")), form="parallel_gated",
            weights_of=None if owner == run else owner, src=i,
            readd_embed=bool(t and i == int(loop["start"]))))
    return out


def gated_layout(l: LayerSpec, width: int
                 ) -> Tuple[Dict[str, Tuple[int, int]], int]:
    """Rows of a gated parallel-form layer's ONE input matrix: every
    projection that reads the normed h — the mixer's (per part, in in_sizes
    order), then the two residual gates 'rg1' (mixer) and 'rg2'
    (feed-forward, when there is one). Every segment starts on a multiple of
    8 rows. Returns ({name: (offset, size)}, total)."""
    ins: Dict[str, Tuple[int, int]] = {}
    a = 0
    for pre, m in mixer_parts(l.mixer):
        for name, n in m.in_sizes:
            ins[pre + name] = (a, n)
            # q, k, v stay neighbours (one conv / one rotation pass)
            a += n if name in ("q", "k") and m.kind == "gqa_attention" \
                else _pad8(n)
    for name in ("rg1", "rg2") if l.ffn is not None else ("rg1",):
        ins[name] = (a, width)
        a += _pad8(width)
    return ins, a


def complete_from_shapes(layers: List[LayerSpec],
                         shapes: Dict[str, Tuple[int, ...]]) -> None:
    """Sizes that only tensor shapes give: the low-rank widths of a delta
    mixer's decay and gate projections ('a1' / 'g1' rows)."""
    for i, l in enumerate(layers):
        src = i if l.weights_of is None else l.weights_of
        m, p = l.mixer, f"l{src}.mix."
        if m.kind == "parallel":
            m, p = m.right, p + "right."
        if m.kind != "delta":
            continue
        if m.channel_decay and p + "a1" in shapes:
            m.decay_rank = int(shapes[p + "a1"][0])
        if m.gate == "sigmoid" and p + "g1" in shapes:
            m.gate_rank = int(shapes[p + "g1"][0])


def _pad8(n: int) -> int:
    return (n + 7) // 8 * 8


def mixer_parts(m) -> List[Tuple[str, Any]]:
    """(tensor-name prefix, sub-mixer) of a mixer: itself, or the two sides
    of a parallel mixer."""
    if m.kind == "parallel":
        return [("left.", m.left), ("right.", m.right)]
    return [("", m)]


def fused_layout(l: LayerSpec) -> Tuple[Dict[str, Tuple[int, int]], int,
                                        Dict[str, Tuple[int, int]], int]:
    """Column layout of a parallel-form layer's two fused GEMMs.
    Input side: every projection that reads the normed h — the mixer's
    (per part, in in_sizes order) and the feed-forward's 'up' — stacked into
    one [rows, width] matrix. Output side: the mixer parts' outputs and the
    feed-forward activation laid side by side as the K axis of one
    [width, K] matrix, so mixer + feed-forward are summed inside the GEMM's
    fp32 accumulator. Every segment starts on a multiple of 8 elements
    (16-byte aligned rows for bf16). Returns (in {name: (offset, size)},
    in_total, out {name: (offset, size)}, out_total)."""
    ins: Dict[str, Tuple[int, int]] = {}
    outs: Dict[str, Tuple[int, int]] = {}
    a = b = 0
    for pre, m in mixer_parts(l.mixer):
        for name, n in m.in_sizes:
            ins[pre + name] = (a, n)
            a += _pad8(n)
        outs[pre + "o"] = (b, m.out_size)
        b += _pad8(m.out_size)
    if l.ffn is not None:
        ins["up"] = (a, l.ffn.ff)
        a += _pad8(l.ffn.ff)
        outs["down"] = (b, l.ffn.ff)
        b += _pad8(l.ffn.ff)
    return ins, a, outs, b


def hybrid_n_params(width: int, vocab: int, taps: int,
                    layers: List[LayerSpec], active_only: bool = False) -> int:
    n = 2 * vocab * width + 1
    for l in layers:
        m = l.mixer
        if l.form == "parallel":
            if l.weights_of is None or active_only:
                n += width + _parallel_layer_params(width, l)
            continue
        if l.form == "sandwich_w":
            if l.weights_of is None or active_only:
                n += _sandwich_w_layer_params(width, l, active_only)
            continue
        if l.form == "parallel_gated":
            if l.weights_of is None or active_only:
                n += _gated_layer_params(width, l, active_only)
            continue
        n += 4 + width * taps
        if m.kind == "latent_attention":
            n += width * (m.q_size + m.cache_dim + m.heads) + m.kv_rank
            n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * width
        else:
            n += width * m.heads * (2 * m.dim + 2 * m.vdim)
            n += m.heads * m.vdim * (1 + width)
        f = l.ffn
        if f is not None:
            e = f.top_k if active_only else f.n_experts
            n += width * f.n_experts + 3 * width * (e * f.ff + f.shared_ff)
    return n


def _sandwich_w_layer_params(width: int, l: LayerSpec,
                             active_only: bool) -> int:
    m, f = l.mixer, l.ffn
    n = 2 * width + width * sum(sz for _, sz in m.in_sizes)
    n += m.heads * m.heads + m.out_size * width
    if isinstance(f, DenseFFNSpec):
        n += 2 * width + 2 * width * f.ff + 4
    elif f is not None:
        e = f.top_k if active_only else f.n_experts
        n += 2 * width + width * f.n_experts + 3 * width * e * f.ff
    return n


def _gated_layer_params(width: int, l: LayerSpec, active_only: bool) -> int:
    n = width + width * (width + 1)                 # norm, mixer gate
    for _, m in mixer_parts(l.mixer):
        n += width * m.out_size
        if m.kind == "latent_attention":
            n += width * (m.cache_dim + m.heads) + m.kv_rank + m.heads
            n += m.kv_rank * m.heads * (m.dim + m.vdim)
            n += (m.q_rank * (width + 1 + m.q_size) if m.q_rank
                  else width * m.q_size)
        elif m.kind == "gqa_attention":
            rows = sum(sz for _, sz in m.in_sizes)
            n += width * rows
            if m.bias:
                n += m.conv_channels + width
            if m.taps > 1:
                n += m.taps * m.conv_channels
            if m.score_mix:
                n += m.heads * m.heads
        else:
            n += 3 * width * m.width + 2 * m.width
    if l.mixer.kind == "parallel" and l.mixer.combine == "normed_mean":
        n += 2 * width
    f = l.ffn
    if f is not None:
        e = f.top_k if active_only else f.n_experts
        n += width * (width + 1) + width * f.n_experts
        n += e * f.ff * width + e * f.up_rows * width
    return n


def _parallel_layer_params(width: int, l: LayerSpec) -> int:
    n = 0
    for _, m in mixer_parts(l.mixer):
        n += width * m.out_size
        if m.kind == "retention":
            n += width * sum(sz for _, sz in m.in_sizes)
        elif m.kind == "sink_attention":
            n += width * sum(sz for _, sz in m.in_sizes) + 2 * m.dim + 2 * m.heads
        else:
            n += (width + m.taps) * m.conv_channels + width * m.heads
            n += m.heads + m.vdim
            hd = m.heads * m.dim
            n += (m.decay_rank * (width + hd) + hd if m.channel_decay
                  else (width + 1) * m.heads)
            hv = m.heads * m.vdim
            n += m.gate_rank * (width + hv) if m.gate_rank else width * hv
    if l.ffn is not None:
        n += 2 * width * l.ffn.ff
    return n


def pugozen_layers(n_layers: int, width: int, *, heads: int = 16,
                   kv_heads: int = 4, dim: int = 128, ff: int = 8192,
                   delta_heads: int = 16, delta_kv_heads: int = 8,
                   delta_dim: int = 128, rank: int = 64, taps: int = 4,
                   side_heads: int = 4, side_dim: int = 64
                   ) -> List[LayerSpec]:
    """A synthetic Pugozen stack for benchmarks: the cycle
    parallel / retention / delta, all with a dense relu^2 feed-forward."""
    out = []
    for i in range(n_layers):
        k = i % 3
        if k == 0:
            mixer: Any = ParallelMixerSpec(
                left=SinkAttnSpec(heads=heads, kv_heads=kv_heads, dim=dim,
                                  vdim=dim, scale=dim ** -0.5, rope_base=1e6,
                                  rope_dims=dim // 2),
                right=DeltaSpec(heads=side_heads, kv_heads=side_heads,
                                dim=side_dim, vdim=side_dim, taps=taps,
                                channel_decay=True, decay_rank=rank,
                                gate="sigmoid", gate_rank=rank),
                left_scale=0.75, right_scale=0.5)
        elif k == 1:
            decay = tuple(1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, heads - 1))
                          for h in range(heads))
            mixer = RetentionSpec(heads=heads, dim=dim, vdim=dim, decay=decay,
                                  rope_base=1e6, rope_dims=dim)
        else:
            mixer = DeltaSpec(heads=delta_heads, kv_heads=delta_kv_heads,
                              dim=delta_dim, vdim=delta_dim, taps=taps)
        out.append(LayerSpec(mixer=mixer, ffn=DenseFFNSpec(ff=ff),
                             form="parallel"))
    return out


def nukopel_layers(n_layers: int, width: int, *, attn_every: int = 4,
                   heads: int = 16, dim: int = 128, rot_dim: int = 64,
                   vdim: int = 128, kv_rank: int = 512, window: int = 4096,
                   li_heads: int = 16, li_dim: int = 128, li_vdim: int = 128,
                   experts: int = 8, top_k: int = 2, ff: int = 2048,
                   shared_ff: int = 2048, limit: float = 7.0
                   ) -> List[LayerSpec]:
    """A synthetic Nukopel stack for benchmarks: lightning layers with a
    latent-attention layer every `attn_every`-th position."""
    out = []
    for i in range(n_layers):
        if (i + 1) % attn_every == 0:
            mixer: Any = LatentAttnSpec(
                heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                kv_rank=kv_rank, window=window, rope_base=1e6,
                rope_dims=rot_dim, scale=(dim + rot_dim) ** -0.5)
        else:
            decay = tuple(1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, li_heads - 1))
                          for h in range(li_heads))
            mixer = LightningSpec(heads=li_heads, dim=li_dim, vdim=li_vdim,
                                  decay=decay)
        out.append(LayerSpec(mixer=mixer, ffn=MoEFFNSpec(
            n_experts=experts, top_k=top_k, ff=ff, limit=limit,
            shared_ff=shared_ff, shared_limit=limit)))
    return out


def pimodra_layers(n_layers: int, width: int, *, heads: int = 16,
                   kv_heads: int = 2, dim: int = 128, window: int = 1024,
                   ff: int = 8192, experts: int = 8, top_k: int = 2,
                   expert_ff: int = 1024, groups: int = 4, keep: int = 2,
                   moe_from: int = 1, loop: Optional[Tuple[int, int, int]] = None
                   ) -> List[LayerSpec]:
    """A synthetic Pimodra stack for benchmarks: head-mixing windowed
    attention everywhere, a dense PolyNorm feed-forward in the layers
    before `moe_from` and group-limited routed experts after; loop =
    (start, stop, times) repeats a block with shared tensors."""
    cfg_layers = []
    for i in range(n_layers):
        mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                 "scale": dim ** -0.5, "mask": {"size": window},
                 "rot": {"base": 1e6, "dims": dim,
                         "scaling": {"factor": 8.0, "original": 4096,
                                     "fast": 32.0, "slow": 1.0}}}
        if i < moe_from:
            mlp: Dict[str, Any] = {"kind": "dense", "ff": ff}
        else:
            mlp = {"kind": "moe", "expert": {"ff": expert_ff},
                   "router": {"experts": experts, "top": top_k,
                              "groups": {"count": groups, "keep": keep}}}
        cfg_layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
    lp = None
    if loop:
        lp = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return looped_layer_specs_from_cfg(cfg_layers, lp)


def zevilorn_layer_cfgs(n_layers: int, width: int, *, heads: int = 16,
                        kv_heads: int = 4, dim: int = 128, window: int = 1024,
                        kv_rank: int = 512, rot_dim: int = 64,
                        q_rank: int = 768, gru_width: Optional[int] = None,
                        experts: int = 8, top_k: int = 2,
                        expert_ff: int = 1024, groups: int = 4, keep: int = 2,
                        taps: int = 4) -> List[Dict[str, Any]]:
    """config.json 'layers' entries of a synthetic Zevilorn stack for
    benchmarks: the cycle capped score-mixing attention / latent attention
    / windowed attention beside a minGRU, every layer with group-routed
    gelu experts."""
    cfg_layers = []
    mlp = {"kind": "moe", "expert": {"ff": expert_ff},
           "router": {"experts": experts, "top": top_k,
                      "groups": {"count": groups, "keep": keep}}}
    for i in range(n_layers):
        k = i % 3
        if k == 0:
            typ = "attention"
            mixer: Dict[str, Any] = {
                "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                "scale": dim ** -0.5, "softcap": 50.0, "conv": taps,
                "mask": {"size": window},
                "rot": {"base": 1e6, "dims": dim,
                        "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                                    "original": 8192}}}
        elif k == 1:
            typ = "latent_attention"
            mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim,
                     "vdim": dim, "kv_rank": kv_rank, "q_rank": q_rank,
                     "scale": (dim + rot_dim) ** -0.5,
                     "rot": {"base": 1e6, "dims": rot_dim}}
        else:
            typ = "parallel"
            mixer = {"left": {"heads": heads, "kv_heads": kv_heads,
                              "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                              "mask": {"size": window},
                              "rot": {"base": 1e6, "dims": dim // 2,
                                      "scaling": {"factor": 2.0}}},
                     "right": {"width": gru_width or width}}
        cfg_layers.append({"type": typ, "mixer": mixer, "mlp": mlp})
    return cfg_layers
