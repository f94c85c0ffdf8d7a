"""Plain, slow CPU statement of the Lidizen decoder, one function per mechanism, in whatever float type the inputs have
(the tests use float64).  TEST INFRASTRUCTURE ONLY: written from the model's equations, shares no code with the product
path, and also makes the random checkpoints the tests load into the product.

Every function sees ONE whole sequence from its first token: no cache, no state, no batching.

The design: token embedding plus a hashed embedding of the (previous, current) token pair, layer-normed; pre-norm layers
whose residual is either one stream or several ("hyper-connections": a sublayer reads a weighted sum of the streams and
its output is spread over a remix of them); the mixer is a softmax attention with grouped key/value heads, biased
projections, an RMS norm over the whole query (key) projection, interleaved rotary pairs on the first dimensions of a
head, scores mixed across heads before the softmax, a sliding window that also keeps the sequence's first tokens, and
values blended with the values of the first such layer; the feed-forward is a biased silu-gated unit or a mixture of
squared-relu experts whose weights are the softmax over the chosen router logits.  The logits use the embedding table.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ------------------------------------------------------------------------------------------------ norms
def layer_norm_ref(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def rms_whole_ref(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the whole last axis (all heads of a projection at once), times ``w``."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


# ------------------------------------------------------------------------------------------------ embedding
def bigram_rows_ref(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the pair table per token: a hash of (previous, current); the first token takes the extra last row."""
    return [buckets if t == 0 else (tokens[t - 1] * mul_prev + tokens[t] * mul_cur) % buckets for t in range(len(tokens))]


def embedding_ref(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype) -> torch.Tensor:
    x = weights["embed"].to(dtype)[torch.tensor(tokens)]
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        rows = bigram_rows_ref(tokens, int(big["buckets"]), int(big["mul_prev"]), int(big["mul_cur"]))
        x = x + weights["bigram"].to(dtype)[torch.tensor(rows)]
    return layer_norm_ref(x, weights["embed.norm"].to(dtype), float(cfg["norm"]["eps"]))


# ------------------------------------------------------------------------------------------------ rotation
def rotate_interleaved_ref(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """``x [T, heads, D]``: pairs (2i, 2i + 1), i < dims / 2, of token t turned by ``t * base^(-2i / dims)``."""
    T = x.shape[0]
    out = x.clone()
    if dims <= 0:
        return out
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ attention
def visible_ref(T: int, size: int, keep_first: int) -> torch.Tensor:
    """``[T, T]`` bool: query i sees key j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def talking_attention_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float,
                          v_first: Optional[torch.Tensor], blend: bool):
    """``h [T, W]`` -> ``(out [T, W], values [T, G, Dv] before blending)``.  ``w``: the mixer's tensors by their short
    names.  ``v_first``: the values of the first blending layer (None in that layer, or without blending)."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = h @ w["q"].T + w["q.b"]
    k = h @ w["k"].T + w["k.b"]
    v = (h @ w["v"].T + w["v.b"]).reshape(T, G, Dv)
    q = rms_whole_ref(q, w["q.norm"], eps).reshape(T, H, D)
    k = rms_whole_ref(k, w["k.norm"], eps).reshape(T, G, D)
    rot = m.get("rot") or {}
    q = rotate_interleaved_ref(q, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))
    k = rotate_interleaved_ref(k, int(rot.get("dims", 0)), float(rot.get("base", 10000.0)))
    v_own = v
    if blend and v_first is not None:
        lam = w["vmix"].reshape(())
        v = (1 - lam) * v + lam * v_first
    scores = torch.empty(H, T, T, dtype=h.dtype)
    for hh in range(H):
        scores[hh] = (q[:, hh] @ k[:, hh // (H // G)].T) * float(m["scale"])
    if "talk" in w:
        scores = torch.einsum("hg,gij->hij", w["talk"], scores)
    mask = m.get("mask") or {}
    vis = visible_ref(T, int(mask.get("size", T + 1)), int(mask.get("keep_first", 0)))
    scores = scores.masked_fill(~vis[None], -math.inf)
    p = torch.softmax(scores, -1)
    o = torch.stack([p[hh] @ v[:, hh // (H // G)] for hh in range(H)], 1).reshape(T, H * Dv)
    return o @ w["o"].T, v_own


# ------------------------------------------------------------------------------------------------ feed-forward
def dense_ff_ref(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    g = h @ w["gate"].T + w["gate.b"]
    u = h @ w["up"].T + w["up.b"]
    return (g * torch.sigmoid(g) * u) @ w["down"].T + w["down.b"]


def moe_ff_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ w["router"].T + w["router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        wt = torch.softmax(z[t, chosen], -1)
        for c, e in enumerate(chosen):
            a = torch.relu(h[t] @ w[f"e{e}.up"].T) ** 2
            out[t] += wt[c] * (a @ w[f"e{e}.down"].T)
    return out


# ------------------------------------------------------------------------------------------------ the model
def _sub(weights: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def lidizen_ref(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
                residuals: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence.  ``residuals`` receives the stream (the sum of the streams) after every layer."""
    eps = float(cfg["norm"]["eps"])
    x0 = embedding_ref(cfg, weights, tokens, dtype)
    S = int(cfg.get("streams") or 0)
    xs = [x0.clone() for _ in range(S)] if S else None
    x = x0
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        for q in (1, 2):
            if q == 2 and layer.get("mlp") is None:
                continue
            hc = _sub(weights, f"{p}hc{q}.", dtype) if S else None
            u = sum(hc["in"][s] * xs[s] for s in range(S)) if S else x
            hn = layer_norm_ref(u, weights[f"{p}norm{q}"].to(dtype), eps)
            if q == 1:
                m = layer["mixer"]
                blend = bool(m.get("v_mix"))
                y, v_own = talking_attention_ref(hn, _sub(weights, p + "mix.", dtype), m, eps, v_first, blend)
                if blend and v_first is None:
                    v_first = v_own
            elif layer["mlp"]["kind"] == "dense":
                y = dense_ff_ref(hn, _sub(weights, p + "mlp.", dtype))
            else:
                y = moe_ff_ref(hn, _sub(weights, p + "mlp.", dtype), layer["mlp"])
            if S:
                xs = [sum(hc["mix"][s, t] * xs[s] for s in range(S)) + hc["out"][t] * y for t in range(S)]
            else:
                x = x + y
        if residuals is not None:
            residuals.append(sum(xs) if S else x.clone())
    if S:
        x = sum(xs)
    return layer_norm_ref(x, weights["final.norm"].to(dtype), eps) @ weights["embed"].to(dtype).T


# ------------------------------------------------------------------------------------------------ random checkpoints
def attention_config(heads=4, kv_heads=2, dim=16, vdim=24, size=12, keep_first=2, rot_dims=8, base=100.0, scale=None, v_mix=True):
    return {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "mask": {"size": size, "keep_first": keep_first},
            "rot": {"base": base, "dims": rot_dims}, "scale": scale if scale is not None else dim ** -0.5, "v_mix": v_mix}


def lidizen_config(vocab=80, width=48, layers=None, streams=3, eps=1e-5, bigram=(53, 7, 5)) -> dict:
    if layers is None:
        layers = [{"type": "attention", "mixer": attention_config(), "mlp": {"kind": "dense", "ff": 72}},
                  {"type": "attention", "mixer": attention_config(), "mlp": {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 6, "top": 2}}}]
    cfg = {"architecture": "Lidizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams:
        cfg["streams"] = streams
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return cfg


def lidizen_random_weights(cfg: dict, seed: int = 0, std: float = 1.0) -> Dict[str, torch.Tensor]:
    """bf16-representable float32 tensors under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    W, V = int(cfg["width"]), int(cfg["vocab"])
    S = int(cfg.get("streams") or 0)

    def rnd(*shape, scale=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * scale * std + mean).to(torch.bfloat16).float()

    w: Dict[str, torch.Tensor] = {"embed": rnd(V, W, scale=0.7), "embed.norm": rnd(W, scale=0.1, mean=1.0), "final.norm": rnd(W, scale=0.1, mean=1.0)}
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        w["bigram"] = rnd(int(big["buckets"]) + 1, W, scale=0.7)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w[p + "norm1"] = rnd(W, scale=0.1, mean=1.0)
        for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
            w[p + "mix." + n] = rnd(rows, W, scale=W ** -0.5)
            w[p + "mix." + n + ".b"] = rnd(rows, scale=0.2)
        w[p + "mix.q.norm"] = rnd(H * D, scale=0.2, mean=1.0)
        w[p + "mix.k.norm"] = rnd(G * D, scale=0.2, mean=1.0)
        w[p + "mix.vmix"] = rnd(1, scale=0.1, mean=0.4).reshape(())
        w[p + "mix.talk"] = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.3 * std).to(torch.bfloat16).float()
        w[p + "mix.o"] = rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
        mlp = layer.get("mlp")
        if mlp is not None:
            w[p + "norm2"] = rnd(W, scale=0.1, mean=1.0)
            if mlp["kind"] == "dense":
                F = mlp["ff"]
                for n in ("gate", "up"):
                    w[p + "mlp." + n] = rnd(F, W, scale=W ** -0.5)
                    w[p + "mlp." + n + ".b"] = rnd(F, scale=0.2)
                w[p + "mlp.down"] = rnd(W, F, scale=F ** -0.5)
                w[p + "mlp.down.b"] = rnd(W, scale=0.2)
            else:
                F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
                for e in range(E):
                    w[f"{p}mlp.e{e}.up"] = rnd(F, W, scale=W ** -0.5)
                    w[f"{p}mlp.e{e}.down"] = rnd(W, F, scale=F ** -0.5)
                w[p + "mlp.router"] = rnd(E, W, scale=W ** -0.5)
                w[p + "mlp.router.b"] = rnd(E, scale=0.3)
        if S:
            for q in (1, 2):
                if q == 2 and mlp is None:
                    continue
                w[f"{p}hc{q}.in"] = rnd(S, scale=0.2, mean=1.0 / S)
                w[f"{p}hc{q}.out"] = rnd(S, scale=0.3, mean=0.7)
                w[f"{p}hc{q}.mix"] = (torch.eye(S) + torch.randn(S, S, generator=g) * 0.15 * std).to(torch.bfloat16).float()
    return w


# ------------------------------------------------------------------------------------------------ kernel-level statements
def shared_key_attention_ref(q: torch.Tensor, rows: torch.Tensor, num_kv_heads: int, v_dim: int, scale: float, first_pos: int,
                             size: Optional[int], keep_first: int) -> torch.Tensor:
    """``q [n, H, Dk]`` are the queries at positions ``first_pos ..``; ``rows [L, Dk + G Dv]`` hold one key for all heads
    followed by the G values.  Query head h reads value ``h // (H / G)``.  Returns ``[n, H, Dv]``."""
    n, H, Dk = q.shape
    L = rows.shape[0]
    keys, vals = rows[:, :Dk], rows[:, Dk:].reshape(L, num_kv_heads, v_dim)
    out = torch.zeros(n, H, v_dim, dtype=q.dtype)
    for r in range(n):
        i = first_pos + r
        js = [j for j in range(i + 1) if size is None or i - j < size or j < keep_first]
        for h in range(H):
            p = torch.softmax((keys[js] @ q[r, h]) * scale, 0)
            out[r, h] = p @ vals[js, h // (H // num_kv_heads)]
    return out


def hyper_step_ref(xs: torch.Tensor, y: Optional[torch.Tensor], mix: torch.Tensor, out_w: torch.Tensor) -> torch.Tensor:
    """``xs [T, S, W]``: every stream rebuilt from the old ones, ``x_t = sum_s mix[s, t] x_s + out_w[t] y``."""
    new = torch.einsum("st,nsw->ntw", mix, xs)
    return new if y is None else new + out_w[None, :, None] * y[:, None, :]
