"""Plain whole-sequence implementation of the Pimodra design, for tests.

One function per mechanism, float64, no cache, no batching, no chunking, and
no code shared with the serving path (bee2bee_amd.*). Inputs: the parsed
config.json dict and a dict of checkpoint-named tensors.

Notation: unit(x) = x / sqrt(mean(x^2) + eps) over the last axis.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int,
               eps: float) -> torch.Tensor:
    """x [T, W]: `groups` equal consecutive parts, each unit-normed on its
    own; the whole row times w."""
    T, W = x.shape
    parts = [unit(x[:, g * (W // groups):(g + 1) * (W // groups)], eps)
             for g in range(groups)]
    return torch.cat(parts, dim=-1) * w


def rope_frequencies(rot: dict):
    """Per-pair angular frequencies and the factor on cos/sin. With a
    'scaling' entry the long-wavelength pairs are slowed by `factor`, the
    short-wavelength ones kept, with a linear ramp between the two pair
    indices that the `fast` and `slow` turn counts over `original`
    positions select."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])

    def pair_index(turns: float) -> float:
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (
            2.0 * math.log(base))

    lo = max(math.floor(pair_index(sc["fast"])), 0)
    hi = min(math.ceil(pair_index(sc["slow"])), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, heads, D]; row t is position t. Coordinate i < dims/2 pairs
    with i + dims/2."""
    T = x.shape[0]
    dims = int(rot["dims"])
    half = dims // 2
    freq, mag = rope_frequencies(rot)
    out = x.clone()
    for t in range(T):
        for i in range(half):
            a = t * freq[i]
            c, s = math.cos(a) * mag, math.sin(a) * mag
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def attention_weights(q: torch.Tensor, k: torch.Tensor, scale: float,
                      window: Optional[int]) -> torch.Tensor:
    """q [T, H, D], k [T, G, D] -> softmax weights [H, T, T] (row i over the
    keys j with 0 <= i - j < window)."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    w = torch.zeros(H, T, T, dtype=F64)
    for h in range(H):
        g = h // rep
        for i in range(T):
            j0 = 0 if not window else max(0, i - window + 1)
            s = (k[j0:i + 1, g] @ q[i, h]) * scale
            e = torch.exp(s - s.max())
            w[h, i, j0:i + 1] = e / e.sum()
    return w


def attention_mixer(h: torch.Tensor, P: Dict[str, torch.Tensor], m: dict,
                    eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
    D, Dv = int(m["dim"]), int(m["vdim"])
    q = (h @ P["q"].T).view(T, H, D)
    k = (h @ P["k"].T).view(T, G, D)
    v = (h @ P["v"].T).view(T, G, Dv)
    if m.get("rot"):
        q, k = rotate(q, m["rot"]), rotate(k, m["rot"])
    q, k = unit(q, eps), unit(k, eps)
    window = (m.get("mask") or {}).get("size")
    w = attention_weights(q, k, float(m["scale"]), window)
    # every head's weights become a mixture of all heads' weights
    w = torch.einsum("hg,gij->hij", P["talk"], w)
    rep = H // G
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        o[:, hh] = w[hh] @ v[:, hh // rep]
    gate = torch.sigmoid(h @ P["g"].T)
    return (o.reshape(T, H * Dv) * gate) @ P["o"].T


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    a, b, c, e = [float(x) for x in coef]
    return a * unit(z, eps) + b * unit(z * z, eps) + c * unit(z ** 3, eps) + e


def dense_ffn(h, P, eps: float):
    return polynorm(h @ P["up"].T, P["act"], eps) @ P["down"].T


def route(h: torch.Tensor, router: torch.Tensor, r: dict):
    """-> (weights [T, E] with zeros for unchosen experts)."""
    T = h.shape[0]
    E, top = int(r["experts"]), int(r["top"])
    z = h @ router.T
    s = torch.softmax(z, dim=-1)
    out = torch.zeros(T, E, dtype=F64)
    grp = r.get("groups") or {"count": 1, "keep": 1}
    n_g, keep = int(grp["count"]), int(grp["keep"])
    per = E // n_g
    for t in range(T):
        gscore = [max(float(s[t, e]) for e in range(g * per, (g + 1) * per))
                  for g in range(n_g)]
        best = sorted(range(n_g), key=lambda g: -gscore[g])[:keep]
        allowed = [e for g in best for e in range(g * per, (g + 1) * per)]
        chosen = sorted(allowed, key=lambda e: -float(s[t, e]))[:top]
        for e in chosen:
            out[t, e] = s[t, e]
    return out


def moe_ffn(h, P, f: dict):
    w = route(h, P["router"], f["router"])
    E = int(f["router"]["experts"])
    y = torch.zeros(h.shape[0], P["e0.down"].shape[0], dtype=F64)
    for e in range(E):
        g = h @ P[f"e{e}.gate"].T
        u = h @ P[f"e{e}.up"].T
        ye = ((g * torch.sigmoid(g)) * u) @ P[f"e{e}.down"].T
        y += w[:, e:e + 1] * ye
    return y


def sub(tensors: Dict[str, torch.Tensor], prefix: str):
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items()
            if k.startswith(prefix)}


def layer_runs(cfg: dict):
    """[(layer index, pass number or None)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int],
            taps: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence. taps: a list that receives
    the residual after every layer run."""
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
    embed = tensors["embed"].to(F64)
    x = embed[torch.tensor(tokens)]
    loop = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t is not None and i == int(loop["start"]):
            x = x + tensors["loop.step"].to(F64)[t]
        l = cfg["layers"][i]
        P = sub(tensors, f"l{i}.")
        if l["type"] != "attention":
            raise ValueError(l["type"])
        y = attention_mixer(group_norm(x, P["norm1"], groups, eps),
                            sub(P, "mix."), l["mixer"], eps)
        x = x + group_norm(y, P["norm1b"], groups, eps)
        f = l.get("mlp")
        if f:
            h = group_norm(x, P["norm2"], groups, eps)
            if f["kind"] == "dense":
                y = dense_ffn(h, sub(P, "mlp."), eps)
            else:
                y = moe_ffn(h, sub(P, "mlp."), f)
            x = x + group_norm(y, P["norm2b"], groups, eps)
        if taps is not None:
            taps.append(x.clone())
    x = group_norm(x, tensors["final.norm"].to(F64), groups, eps)
    return x @ embed.T


# ------------------------------------------------ small random checkpoints

def make_config(vocab=97, width=24, groups=2, eps=1e-6, heads=4, kv_heads=2,
                dim=6, vdim=10, window=9, rot_dims=4, scaling=True,
                kinds=("dense", "moe", "moe"), ff=20, experts=6, top=2,
                n_groups=3, keep=2, expert_ff=8, loop=(1, 3, 2)) -> dict:
    rot = None
    if rot_dims:
        rot = {"base": 500.0, "dims": rot_dims}
        if scaling:
            rot["scaling"] = {"factor": 3.0, "original": 16, "fast": 4.0,
                              "slow": 0.5}
    layers = []
    for kind in kinds:
        mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                 "vdim": vdim, "scale": 1.7 / math.sqrt(dim)}
        if window:
            mixer["mask"] = {"size": window}
        if rot:
            mixer["rot"] = rot
        if kind == "dense":
            mlp = {"kind": "dense", "ff": ff}
        elif kind == "moe":
            mlp = {"kind": "moe", "expert": {"ff": expert_ff},
                   "router": {"experts": experts, "top": top,
                              "groups": {"count": n_groups, "keep": keep}}}
        else:
            mlp = None
        layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Pimodra", "vocab": vocab, "width": width,
           "norm": {"eps": eps, "groups": groups}, "layers": layers}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bf16 tensors under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    W = int(cfg["width"])

    def rnd(*shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(*shape, generator=g)).bfloat16()

    T = {"embed": rnd(cfg["vocab"], W), "final.norm": rnd(W, std=0.1, mean=1.0)}
    if cfg.get("loop"):
        T["loop.step"] = rnd(int(cfg["loop"]["times"]), W, std=0.5)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        H, G = m["heads"], m.get("kv_heads", m["heads"])
        D, Dv = m["dim"], m["vdim"]
        for n in ("norm1", "norm1b"):
            T[p + n] = rnd(W, std=0.1, mean=1.0)
        T[p + "mix.q"] = rnd(H * D, W, std=W ** -0.5)
        T[p + "mix.k"] = rnd(G * D, W, std=W ** -0.5)
        T[p + "mix.v"] = rnd(G * Dv, W, std=W ** -0.5)
        T[p + "mix.g"] = rnd(H * Dv, W, std=W ** -0.5)
        T[p + "mix.o"] = rnd(W, H * Dv, std=(H * Dv) ** -0.5)
        T[p + "mix.talk"] = (torch.eye(H) + 0.3 * torch.randn(
            H, H, generator=g)).bfloat16()
        f = l.get("mlp")
        if not f:
            continue
        for n in ("norm2", "norm2b"):
            T[p + n] = rnd(W, std=0.1, mean=1.0)
        if f["kind"] == "dense":
            T[p + "mlp.up"] = rnd(f["ff"], W, std=W ** -0.5)
            T[p + "mlp.down"] = rnd(W, f["ff"], std=f["ff"] ** -0.5)
            T[p + "mlp.act"] = rnd(4, std=0.3, mean=0.3)
        else:
            ff = f["expert"]["ff"]
            T[p + "mlp.router"] = rnd(f["router"]["experts"], W, std=1.5 * W ** -0.5)
            for e in range(f["router"]["experts"]):
                T[f"{p}mlp.e{e}.gate"] = rnd(ff, W, std=W ** -0.5)
                T[f"{p}mlp.e{e}.up"] = rnd(ff, W, std=W ** -0.5)
                T[f"{p}mlp.e{e}.down"] = rnd(W, ff, std=ff ** -0.5)
    return T


def save_checkpoint(path: str, cfg: dict, tensors: Dict[str, torch.Tensor]):
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    save_file({k: v.contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
