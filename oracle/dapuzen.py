"""Plain, slow CPU statement of the Dapuzen decoder, one function per mechanism, in whatever float type the inputs
have (the tests use float64).  TEST INFRASTRUCTURE ONLY: written from the model's equations, shares no code with the
product path, and also makes the random checkpoints the tests load into the product.

Every function sees ONE whole sequence from its first token: no cache, no state, no batching.

The design: a decoder of parallel layers (``h = norm(x); x <- x + mixer(h) + ff(h)``, the norm an RMS norm times ONE
number) on a scaled embedding.  Mixers: a windowed softmax attention with grouped key/value heads, half-split rotary
pairs and a sigmoid gate per head; a retention (linear attention with a constant decay per head, rotary queries and keys,
unit-RMS heads, silu gate); or two mixers side by side on the same input, a windowed attention with biases and
tanh-capped scores and no rotation beside a Mamba-2 state-space layer, summed with two constants.  Feed-forwards: dense
(xIELU) or a mixture of silu-gated experts whose router is a softmax over experts and identity experts, chosen by
corrected scores within the best groups, beside a shared expert behind a sigmoid gate of one number per token.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F


# ------------------------------------------------------------------------------------------------ norms
def unit_rms_ref(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm_ref(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm times the single number ``g``."""
    return unit_rms_ref(x, eps) * g.reshape(())


# ------------------------------------------------------------------------------------------------ rotation
def rotate_half_ref(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """``x [T, heads, D]``: of every head's first ``dims`` dimensions, i and i + dims / 2 turn together by
    ``t * base^(-2 i / dims)``; the rest pass."""
    if not dims:
        return x
    T, half = x.shape[0], dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# ------------------------------------------------------------------------------------------------ softmax attention
def window_attention_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int],
                         softcap: Optional[float] = None) -> torch.Tensor:
    """``q [T, H, D]``, ``k [T, G, D]``, ``v [T, G, Dv]`` -> ``[T, H, Dv]``: query i sees keys j with
    ``0 <= i - j < window``; scores ``scale q.k``, then ``softcap tanh(score / softcap)``."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window is None else max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            out[i, h] = torch.softmax(s, 0) @ v[lo:i + 1, g]
    return out


def gated_attention_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """The 'attention' mixer: rotary queries and keys, window, a sigmoid gate per head on the heads' outputs."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    q = rotate_half_ref((h @ w["q"].T).view(T, H, D), rot.get("dims", 0), rot.get("base", 10000.0))
    k = rotate_half_ref((h @ w["k"].T).view(T, G, D), rot.get("dims", 0), rot.get("base", 10000.0))
    v = (h @ w["v"].T).view(T, G, Dv)
    o = window_attention_ref(q, k, v, m["scale"], (m.get("mask") or {}).get("size"))
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * Dv) @ w["o"].T


def capped_attention_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """The left half of the 'parallel' mixer: biased projections, no rotation, tanh-capped scores, window."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).view(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, D)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, Dv)
    o = window_attention_ref(q, k, v, m["scale"], (m.get("mask") or {}).get("size"), m.get("softcap"))
    return o.reshape(T, H * Dv) @ w["o"].T + w["o.b"]


# ------------------------------------------------------------------------------------------------ state-space layer
def causal_conv_ref(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """``x [T, C]``, ``w [C, taps]`` (the last column weighs the current token), zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], 0)
    out = b.expand(T, -1).clone()
    for j in range(taps):
        out = out + pad[j:j + T] * w[:, j]
    return out


def ssd_scan_ref(x: torch.Tensor, dt: torch.Tensor, a_log: torch.Tensor, B: torch.Tensor, C: torch.Tensor, D: torch.Tensor) -> torch.Tensor:
    """``x [T, H, P]``, ``dt [T, H]`` (after softplus), ``B, C [T, G, N]`` -> ``y [T, H, P]`` with
    ``S_t = exp(-exp(a_log) dt_t) S_{t-1} + dt_t B_t x_t^T`` (``S [N, P]``) and ``y_t = S_t^T C_t + D x_t``."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    y = torch.zeros_like(x)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(N, P, dtype=x.dtype)
        for t in range(T):
            S = torch.exp(-torch.exp(a_log[h]) * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


def mamba2_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """The right half of the 'parallel' mixer."""
    T = h.shape[0]
    H, P, N, G, NG = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * P
    proj = h @ w["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = F.silu(causal_conv_ref(xbc, w["conv"], w["conv.b"]))
    x, B, C = xbc[:, :inner].view(T, H, P), xbc[:, inner:inner + G * N].view(T, G, N), xbc[:, inner + G * N:].view(T, G, N)
    dt = F.softplus(dt + w["dt_bias"])
    y = ssd_scan_ref(x, dt, w["A_log"], B, C, w["D"]).reshape(T, inner)
    y = y * F.silu(z)
    y = unit_rms_ref(y.view(T, NG, inner // NG), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T


def parallel_mixer_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    left = capped_attention_ref(h, {k[5:]: v for k, v in w.items() if k.startswith("left.")}, m["left"])
    right = mamba2_ref(h, {k[6:]: v for k, v in w.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ------------------------------------------------------------------------------------------------ retention
def retention_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    q = rotate_half_ref((h @ w["q"].T).view(T, H, D), rot.get("dims", 0), rot.get("base", 10000.0))
    k = rotate_half_ref((h @ w["k"].T).view(T, H, D), rot.get("dims", 0), rot.get("base", 10000.0)) * D ** -0.5
    v = (h @ w["v"].T).view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = m["decay"][hh] * S + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    o = unit_rms_ref(o, eps).reshape(T, H * Dv) * F.silu(h @ w["g"].T)
    return o @ w["o"].T


# ------------------------------------------------------------------------------------------------ feed-forward
def xielu_ref(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    pos = F.softplus(p) * z * z + z / 2
    neg = (0.5 + F.softplus(q)) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ff_ref(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return xielu_ref(h @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


def silu_expert_ref(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (F.silu(h @ gate.T) * (h @ up.T)) @ down.T


def grouped_route_ref(logits: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """``logits [T, E]`` -> ``(chosen [T, top], weights [T, top])``: softmax scores; the choice goes by score + correction
    among the experts of the ``keep`` groups (of ``groups`` equal runs of neighbours) whose best corrected score is largest;
    the weights are the uncorrected scores."""
    T, E = logits.shape
    s = torch.softmax(logits, -1)
    c = s + correction
    best = c.view(T, groups, E // groups).max(-1).values
    kept = torch.zeros(T, groups, dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    c = torch.where(kept[:, :, None].expand(T, groups, E // groups).reshape(T, E), c, torch.full_like(c, -math.inf))
    chosen = c.topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen)


def moe_ff_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    grp = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weights = grouped_route_ref(h @ w["router"].T, w["correction"], top, grp["count"], grp["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t].tolist(), weights[t]):
            if e >= E:
                out[t] = out[t] + wt * h[t]                 # an identity expert
            else:
                out[t] = out[t] + wt * silu_expert_ref(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if mlp.get("shared"):
        sh = silu_expert_ref(h, w["shared.gate"], w["shared.up"], w["shared.down"])
        out = out + sh * torch.sigmoid(h @ w["shared.sg"].T)
    return out


# ------------------------------------------------------------------------------------------------ the model
def _sub(weights: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def mixer_ref(kind: str, h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    if kind == "attention":
        return gated_attention_ref(h, w, m)
    if kind == "retention":
        return retention_ref(h, w, m, eps)
    if kind == "parallel":
        return parallel_mixer_ref(h, w, m, eps)
    raise ValueError(kind)


def dapuzen_ref(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
                residual_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence."""
    eps = cfg["norm"]["eps"]
    x = weights["embed"].to(dtype)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{entry.get('weights_of', i)}."
        h = scalar_norm_ref(x, weights[p + "norm1"].to(dtype), eps)
        y = mixer_ref(entry["type"], h, _sub(weights, p + "mix.", dtype), entry["mixer"], eps)
        if entry.get("mlp") is not None:
            fw = _sub(weights, p + "mlp.", dtype)
            y = y + (dense_ff_ref(h, fw) if entry["mlp"]["kind"] == "dense" else moe_ff_ref(h, fw, entry["mlp"]))
        x = x + y
        if residual_out is not None:
            residual_out.append(x.clone())
    x = scalar_norm_ref(x, weights["final.norm"].to(dtype), eps)
    return x @ weights["head"].to(dtype).T


# ------------------------------------------------------------------------------------------------ test checkpoints
def attention_mixer_config(heads=6, kv_heads=2, dim=24, vdim=40, window=13, rot_dims=16, base=10000.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(scale if scale is not None else dim ** -0.5)}
    if window is not None:
        m["mask"] = {"size": window}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return m


def retention_mixer_config(heads=3, dim=16, vdim=24, rot_dims=8, base=5000.0, decay=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay) if decay is not None else [1 - 2.0 ** (-3 - h) for h in range(heads)]}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return m


def parallel_mixer_config(heads=4, kv_heads=2, dim=16, vdim=24, window=9, softcap=3.0, ssm_heads=6, ssm_vdim=8, state=12, groups=3,
                          norm_groups=2, conv=3, left_scale=0.8, right_scale=1.3):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": softcap}
    if window is not None:
        left["mask"] = {"size": window}
    right = {"heads": ssm_heads, "vdim": ssm_vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def moe_config(experts=5, identity=3, top=3, groups=4, keep=2, ff=24, shared_ff=40):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top,
                                                            "groups": {"count": groups, "keep": keep}}}
    if shared_ff:
        mlp["shared"] = {"ff": shared_ff}
    return mlp


def dapuzen_config(vocab=96, width=48, layers=None, eps=1e-5, embed_scale=3.0) -> dict:
    """``layers``: a list of ``(type, mixer config, mlp config or None)`` or ``("weights_of", j)``."""
    if layers is None:
        layers = [("attention", attention_mixer_config(), {"kind": "dense", "ff": 72}),
                  ("parallel", parallel_mixer_config(), moe_config()),
                  ("retention", retention_mixer_config(), None),
                  ("weights_of", 1),
                  ("attention", attention_mixer_config(heads=4, kv_heads=4, dim=16, vdim=16, window=None, rot_dims=8), moe_config(shared_ff=0))]
    out = []
    for entry in layers:
        if entry[0] == "weights_of":
            src = dict(out[entry[1]])
            src["weights_of"] = entry[1]
            out.append(src)
        else:
            out.append({"type": entry[0], "mixer": entry[1], "mlp": entry[2]})
    return {"architecture": "Dapuzen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
            "layers": out}


def dapuzen_random_weights(cfg: dict, seed: int = 0, std: float = 1.0) -> Dict[str, torch.Tensor]:
    """bf16-representable random tensors under the checkpoint's names (fp32 tensors whose values survive a bf16 round trip)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rnd(*shape, s=1.0):
        return (torch.randn(shape, generator=g) * s * std).to(torch.bfloat16).float()

    def lin(o, i):
        return rnd(o, i, s=i ** -0.5)

    def attention(p, m, biased, gated):
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        w[p + "q"], w[p + "k"], w[p + "v"], w[p + "o"] = lin(H * D, W), lin(G * D, W), lin(G * Dv, W), lin(W, H * Dv)
        if biased:
            w[p + "q.b"], w[p + "k.b"], w[p + "v.b"], w[p + "o.b"] = rnd(H * D, s=0.2), rnd(G * D, s=0.2), rnd(G * Dv, s=0.2), rnd(W, s=0.2)
        if gated:
            w[p + "g"] = lin(H, W)

    w: Dict[str, torch.Tensor] = {"embed": rnd(cfg["vocab"], W, s=1.0 / cfg["embedding"]["scale"]), "head": lin(cfg["vocab"], W),
                                  "final.norm": 1 + rnd(s=0.1)}
    for i, entry in enumerate(cfg["layers"]):
        if "weights_of" in entry:
            continue
        p, m = f"l{i}.", entry["mixer"]
        w[p + "norm1"] = 1 + rnd(s=0.1)
        if entry["type"] == "attention":
            attention(p + "mix.", m, False, True)
        elif entry["type"] == "retention":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = lin(H * D, W), lin(H * D, W), lin(H * Dv, W)
            w[p + "mix.g"], w[p + "mix.o"] = lin(H * Dv, W), lin(W, H * Dv)
        else:
            attention(p + "mix.left.", m["left"], True, False)
            r = m["right"]
            H, P, N, G = r["heads"], r["vdim"], r["state"], r["groups"]
            inner, ch = H * P, H * P + 2 * G * N
            q = p + "mix.right."
            w[q + "in"], w[q + "conv"], w[q + "conv.b"] = lin(2 * inner + 2 * G * N + H, W), rnd(ch, r["conv"], s=r["conv"] ** -0.5), rnd(ch, s=0.1)
            w[q + "dt_bias"], w[q + "A_log"], w[q + "D"] = rnd(H, s=0.5), rnd(H, s=0.5) - 1.0, 1 + rnd(H, s=0.2)
            w[q + "norm"], w[q + "o"] = 1 + rnd(inner, s=0.1), lin(W, inner)
        mlp = entry.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            Fd = mlp["ff"]
            w[p + "mlp.up"], w[p + "mlp.down"], w[p + "mlp.act"] = lin(Fd, W), lin(W, Fd), rnd(2)
        else:
            Fe, r = mlp["expert"]["ff"], mlp["router"]
            for e in range(r["experts"]):
                w[f"{p}mlp.e{e}.gate"], w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = lin(Fe, W), lin(Fe, W), lin(W, Fe)
            n = r["experts"] + r.get("identity", 0)
            w[p + "mlp.router"], w[p + "mlp.correction"] = rnd(n, W, s=2.0 * W ** -0.5), rnd(n, s=0.1)
            if mlp.get("shared"):
                Fs = mlp["shared"]["ff"]
                w[p + "mlp.shared.gate"], w[p + "mlp.shared.up"], w[p + "mlp.shared.down"] = lin(Fs, W), lin(Fs, W), lin(W, Fs)
                w[p + "mlp.shared.sg"] = lin(1, W)
    return w
