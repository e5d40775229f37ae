"""Plain whole-sequence implementation of the Zevilorn design, for tests.

One function per mechanism, float64, no cache, no batching, no chunking, and
no code shared with the serving path (bee2bee_amd.*). Inputs: the parsed
config.json dict and a dict of checkpoint-named tensors.

Notation: unit(x) = x / sqrt(mean(x^2) + eps) over the last axis; row t of a
[T, ...] tensor is position t of one sequence.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def linear(W: Dict[str, torch.Tensor], name: str, x: torch.Tensor,
           bias: bool = False) -> torch.Tensor:
    y = x @ W[name].double().t()
    if bias:
        y = y + W[name + ".b"].double()
    return y


# ------------------------------------------------------------- rotation

def frequencies(rot: dict, rule: str) -> List[float]:
    """Angular frequency of every rotated pair. rule "banded": pairs whose
    wavelength exceeds original/low are slowed by `factor`, those shorter
    than original/high are kept, a linear blend between. rule "linear":
    every pair is slowed by `factor`. No 'scaling' entry: as they are."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f
    factor = float(sc["factor"])
    if rule == "linear":
        return [x / factor for x in f]
    lo, hi, orig = float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = []
    for x in f:
        wl = 2.0 * math.pi / x
        if wl < orig / hi:
            out.append(x)
        elif wl > orig / lo:
            out.append(x / factor)
        else:
            s = (orig / wl - lo) / (hi - lo)
            out.append((1.0 - s) * x / factor + s * x)
    return out


def rotate(x: torch.Tensor, freq: List[float], layout: str) -> torch.Tensor:
    """x [T, heads, D]. layout "interleaved": coordinate 2i pairs with 2i+1;
    "half": coordinate i pairs with i + n, n = number of pairs. Coordinates
    past the rotated ones pass."""
    n = len(freq)
    out = x.clone()
    pos = torch.arange(x.shape[0], dtype=F64)
    for i in range(n):
        a = pos * freq[i]
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        ia, ib = (2 * i, 2 * i + 1) if layout == "interleaved" else (i, i + n)
        u, v = x[:, :, ia], x[:, :, ib]
        out[:, :, ia] = u * c - v * s
        out[:, :, ib] = v * c + u * s
    return out


# ----------------------------------------------------------- attention

def short_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros
    before the start."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def visible(T: int, window: Optional[int]) -> torch.Tensor:
    i = torch.arange(T)
    d = i[:, None] - i[None, :]
    ok = d >= 0
    if window:
        ok = ok & (d < window)
    return ok


def softmax_rows(s: torch.Tensor, ok: torch.Tensor,
                 extra: Optional[torch.Tensor]) -> torch.Tensor:
    """s [H, T, T], ok [T, T]; extra [H] or None: a logit per head that
    counts once in the denominator and has no value."""
    s = s.masked_fill(~ok[None], float("-inf"))
    m = s.max(-1, keepdim=True).values
    if extra is not None:
        m = torch.maximum(m, extra.view(-1, 1, 1))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if extra is not None:
        den = den + torch.exp(extra.view(-1, 1, 1) - m)
    return e / den


def gqa_scores(q: torch.Tensor, k: torch.Tensor, scale: float) -> torch.Tensor:
    """q [T, H, D], k [T, G, D] -> [H, T, T]."""
    H, G = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    return torch.einsum("ihd,jhd->hij", q, kk) * scale


def gqa_apply(p: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """p [H, T, T], v [T, G, Dv] -> [T, H * Dv]."""
    H, G = p.shape[0], v.shape[1]
    vv = v.repeat_interleave(H // G, dim=1)
    return torch.einsum("hij,jhd->ihd", p, vv).reshape(p.shape[1], -1)


def capped_attention(W, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
    """Biased projections, a short conv on each, interleaved rotation with
    banded scaling, capped scores mixed across heads, window, a zero logit
    in the denominator."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = linear(W, p + "q", h, True)
    k = linear(W, p + "k", h, True)
    v = linear(W, p + "v", h, True)
    if m.get("conv"):
        q = short_conv(q, W[p + "q.conv"].double())
        k = short_conv(k, W[p + "k.conv"].double())
        v = short_conv(v, W[p + "v.conv"].double())
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, Dv)
    if m.get("rot"):
        f = frequencies(m["rot"], "banded")
        q, k = rotate(q, f, "interleaved"), rotate(k, f, "interleaved")
    s = gqa_scores(q, k, float(m["scale"]))
    cap = m.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    s = torch.einsum("hg,gij->hij", W[p + "talk"].double(), s)
    ok = visible(T, (m.get("mask") or {}).get("size"))
    pr = softmax_rows(s, ok, torch.zeros(H, dtype=F64))
    return linear(W, p + "o", gqa_apply(pr, v), True)


def latent_attention(W, p: str, m: dict, h: torch.Tensor,
                     eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, R, Dv, C = (int(m["heads"]), int(m["dim"]), int(m["rot_dim"]),
                      int(m["vdim"]), int(m["kv_rank"]))
    cq = unit(linear(W, p + "dq", h), eps) * W[p + "dq.norm"].double()
    q = linear(W, p + "uq", cq).view(T, H, D + R)
    dkv = linear(W, p + "dkv", h)
    c = unit(dkv[:, :C], eps) * W[p + "dkv.norm"].double()
    f = frequencies(dict(m["rot"], scaling=None), "none")
    kr = rotate(dkv[:, C:].reshape(T, 1, R), f, "half")          # [T, 1, R]
    qr = rotate(q[..., D:].contiguous(), f, "half")
    kn = linear(W, p + "uk", c).view(T, H, D)
    v = linear(W, p + "uv", c).view(T, H, Dv)
    s = torch.einsum("ihd,jhd->hij", q[..., :D], kn)
    s = s + torch.einsum("ihr,jr->hij", qr, kr[:, 0])
    s = s * float(m["scale"])
    pr = softmax_rows(s, visible(T, None), W[p + "sink"].double())
    o = torch.einsum("hij,jhd->ihd", pr, v)
    o = o * sigmoid(linear(W, p + "g", h))[..., None]
    return linear(W, p + "o", o.reshape(T, H * Dv))


def windowed_attention(W, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
    """The left side of a parallel mixer."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = linear(W, p + "q", h).view(T, H, D)
    k = linear(W, p + "k", h).view(T, G, D)
    v = linear(W, p + "v", h).view(T, G, Dv)
    if m.get("rot"):
        f = frequencies(m["rot"], "linear")
        q, k = rotate(q, f, "interleaved"), rotate(k, f, "interleaved")
    s = gqa_scores(q, k, float(m["scale"]))
    pr = softmax_rows(s, visible(T, (m.get("mask") or {}).get("size")), None)
    o = gqa_apply(pr, v).view(T, H, Dv)
    o = o * sigmoid(linear(W, p + "g", h))[..., None]
    return linear(W, p + "o", o.reshape(T, H * Dv))


def min_gru(W, p: str, h: torch.Tensor) -> torch.Tensor:
    """The right side of a parallel mixer: S_t = (1 - z) S_(t-1) + z c_t."""
    z = sigmoid(linear(W, p + "z", h, True))
    u = linear(W, p + "x", h, True)
    cand = torch.where(u >= 0, u + 0.5, sigmoid(u))
    g = linear(W, p + "g", h)
    S = torch.zeros(u.shape[1], dtype=F64)
    rows = []
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        rows.append(S * (g[t] * sigmoid(g[t])))
    return linear(W, p + "o", torch.stack(rows))


def parallel_mixer(W, p: str, m: dict, h: torch.Tensor,
                   eps: float) -> torch.Tensor:
    a = windowed_attention(W, p + "left.", m["left"], h)
    b = min_gru(W, p + "right.", h)
    return 0.5 * (unit(a, eps) * W[p + "left.out"].double()
                  + unit(b, eps) * W[p + "right.out"].double())


# --------------------------------------------------------- feed-forward

def route(z: torch.Tensor, r: dict):
    """z [E] router logits -> (chosen expert indices, their weights)."""
    E, top = int(r["experts"]), int(r["top"])
    s = sigmoid(z)
    g = r.get("groups") or {}
    n_g = int(g.get("count", 1))
    keep = int(g.get("keep", n_g))
    size = E // n_g
    gscore = []
    for a in range(n_g):
        part = sorted(s[a * size:(a + 1) * size].tolist(), reverse=True)
        gscore.append(sum(part[:2]))
    kept = sorted(range(n_g), key=lambda a: (-gscore[a], a))[:keep]
    cand = [e for e in range(E) if e // size in kept]
    cand.sort(key=lambda e: (-float(s[e]), e))
    chosen = cand[:top]
    return chosen, [s[e] for e in chosen]


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def experts(W, p: str, f: dict, h: torch.Tensor) -> torch.Tensor:
    z = linear(W, p + "router", h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, wts = route(z[t], f["router"])
        for e, w in zip(chosen, wts):
            a = gelu_erf(W[f"{p}e{e}.up"].double() @ h[t])
            out[t] += w * (W[f"{p}e{e}.down"].double() @ a)
    return out


# --------------------------------------------------------------- model

def run_order(cfg: dict) -> List[tuple]:
    """[(checkpoint layer, first of a later pass?)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(a)]
    for t in range(times):
        order += [(i, t > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def layer(W, i: int, l: dict, x: torch.Tensor, eps: float) -> torch.Tensor:
    p = f"l{i}."
    h = unit(x, eps) * W[p + "norm1"].double()
    m = l["mixer"]
    if l["type"] == "attention":
        y = capped_attention(W, p + "mix.", m, h)
    elif l["type"] == "latent_attention":
        y = latent_attention(W, p + "mix.", m, h, eps)
    else:
        y = parallel_mixer(W, p + "mix.", m, h, eps)
    out = x + y * sigmoid(linear(W, p + "rg1", h, True))
    if l.get("mlp"):
        f = experts(W, p + "mlp.", l["mlp"], h)
        out = out + f * sigmoid(linear(W, p + "rg2", h, True))
    return out


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int],
            residuals: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab]; residuals (a list) receives the stream after every
    layer run."""
    eps = float(cfg["norm"]["eps"])
    e0 = W["embed"].double()[torch.tensor(tokens)]
    x = e0.clone()
    for i, again in run_order(cfg):
        if again:
            x = x + e0
        x = layer(W, i, cfg["layers"][i], x, eps)
        if residuals is not None:
            residuals.append(x.clone())
    x = unit(x, eps) * W["final.norm"].double()
    return x @ W["head"].double().t()


# ------------------------------------------------- random checkpoints

def make_config(vocab=61, width=24, kinds=("attention", "latent_attention",
                                           "parallel"),
                loop=(1, 3, 2), heads=4, kv_heads=2, dim=6, vdim=10,
                window=9, rot_dims=4, scaling=True, softcap=2.5, conv=3,
                lat_heads=3, lat_dim=6, rot_dim=4, lat_vdim=5, kv_rank=7,
                q_rank=9, left_heads=4, left_kv=2, left_dim=8, left_vdim=6,
                left_window=7, left_rot=4, gru=13, experts=8, top=3,
                n_groups=4, keep=3, ff=10, no_mlp=(), eps=1e-5):
    """A small config of the design; `kinds` lists the layers, `no_mlp` the
    indices of layers without a feed-forward, loop = (start, stop, times)."""
    layers = []
    for i, kind in enumerate(kinds):
        if kind == "attention":
            rot = {"base": 500.0, "dims": rot_dims}
            if scaling:
                rot["scaling"] = {"factor": 4.0, "low": 1.0, "high": 4.0,
                                  "original": 16}
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                     "vdim": vdim, "scale": dim ** -0.5, "softcap": softcap,
                     "conv": conv, "mask": {"size": window}}
            if rot_dims:
                mixer["rot"] = rot
        elif kind == "latent_attention":
            mixer = {"heads": lat_heads, "dim": lat_dim, "rot_dim": rot_dim,
                     "vdim": lat_vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                     "scale": (lat_dim + rot_dim) ** -0.5,
                     "rot": {"base": 300.0, "dims": rot_dim}}
        else:
            left = {"heads": left_heads, "kv_heads": left_kv, "dim": left_dim,
                    "vdim": left_vdim, "scale": left_dim ** -0.5,
                    "mask": {"size": left_window}}
            if left_rot:
                left["rot"] = {"base": 100.0, "dims": left_rot,
                               "scaling": {"factor": 2.0}}
            mixer = {"left": left, "right": {"width": gru}}
        mlp = None if i in no_mlp else {
            "kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top,
                       "groups": {"count": n_groups, "keep": keep}}}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Zevilorn", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "layers": layers}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    Wd, V = int(cfg["width"]), int(cfg["vocab"])
    out = {"embed": (V, Wd), "final.norm": (Wd,), "head": (V, Wd)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        out[p + "norm1"] = (Wd,)
        out[p + "rg1"], out[p + "rg1.b"] = (Wd, Wd), (Wd,)
        if l["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n_, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                out[p + "mix." + n_] = (rows, Wd)
                out[p + "mix." + n_ + ".b"] = (rows,)
                if m.get("conv"):
                    out[p + "mix." + n_ + ".conv"] = (rows, m["conv"])
            out[p + "mix.talk"] = (H, H)
            out[p + "mix.o"], out[p + "mix.o.b"] = (Wd, H * Dv), (Wd,)
        elif l["type"] == "latent_attention":
            H, D, R, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            C, Q = m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (Q, Wd), p + "mix.dq.norm": (Q,),
                        p + "mix.uq": (H * (D + R), Q),
                        p + "mix.dkv": (C + R, Wd), p + "mix.dkv.norm": (C,),
                        p + "mix.uk": (H * D, C), p + "mix.uv": (H * Dv, C),
                        p + "mix.sink": (H,), p + "mix.g": (H, Wd),
                        p + "mix.o": (Wd, H * Dv)})
        else:
            a, b = m["left"], m["right"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            out.update({p + "mix.left.q": (H * D, Wd),
                        p + "mix.left.k": (G * D, Wd),
                        p + "mix.left.v": (G * Dv, Wd),
                        p + "mix.left.g": (H, Wd),
                        p + "mix.left.o": (Wd, H * Dv),
                        p + "mix.left.out": (Wd,), p + "mix.right.out": (Wd,)})
            n = b["width"]
            out.update({p + "mix.right.z": (n, Wd), p + "mix.right.z.b": (n,),
                        p + "mix.right.x": (n, Wd), p + "mix.right.x.b": (n,),
                        p + "mix.right.g": (n, Wd), p + "mix.right.o": (Wd, n)})
        f = l.get("mlp")
        if f:
            out[p + "rg2"], out[p + "rg2.b"] = (Wd, Wd), (Wd,)
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            out[p + "mlp.router"] = (E, Wd)
            for e in range(E):
                out[f"{p}mlp.e{e}.up"] = (ff, Wd)
                out[f"{p}mlp.e{e}.down"] = (Wd, ff)
    return out


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bf16-representable random tensors under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        t = torch.randn(shape, generator=g)
        last = name.split(".")[-1]
        if last in ("norm1", "norm", "out") or name == "final.norm":
            t = 1.0 + 0.2 * t
        elif name in ("embed",):
            t = t
        elif last == "conv":
            t = 0.5 * t
        elif last == "talk":
            t = torch.eye(shape[0]) + 0.3 * t
        elif last in ("b", "sink"):
            t = 0.5 * t
        elif last == "router":
            t = t * (2.0 / math.sqrt(shape[-1]))
        else:
            t = t * (1.5 / math.sqrt(shape[-1]))
        W[name] = t.bfloat16().float()
    return W


def save_checkpoint(path: str, cfg: dict, W: Dict[str, torch.Tensor]) -> None:
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
