"""A plain float64 formulation of the Zusotar design, one function per mechanism, written from the design's equations.
It shares no code with the product path: whole sequences, explicit loops over tokens where a recurrence runs, dense
score matrices with explicit masks. Weights arrive as a dict of float64 tensors under the checkpoint's names.

Notation: W width, H heads, G key/value heads, D key size, V value size, R latent size, P rotated size, n tokens.
"""
import math
from typing import Any, Dict, List, Optional, Tuple

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_centered(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Rotate the first `dims` coordinates of x [n, ..., d]: coordinate 2i with 2i + 1 by the angle pos * base^(-2i/dims)."""
    out = x.clone()
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        a = pos.to(F64) * f
        shape = (x.shape[0],) + (1,) * (x.dim() - 2)
        c, s = torch.cos(a).reshape(shape), torch.sin(a).reshape(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def embedding(tokens: List[int], w: Dict[str, torch.Tensor], start: int = 0) -> torch.Tensor:
    pos = torch.arange(start, start + len(tokens))
    return w["embed"][torch.tensor(tokens)] + w["pos"][pos]


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Causal attention through a shared latent with one sink logit per head in the denominator."""
    n = h.shape[0]
    H, D, P, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    q = (h @ w[p + "q"].T).view(n, H, D + P)
    dkv = h @ w[p + "dkv"].T
    c = norm_plain(dkv[:, :R], w[p + "dkv.norm"], eps)
    kr = rotate_pairs(dkv[:, R:R + P], pos, m["rot"]["base"], m["rot"]["dims"])
    qr = rotate_pairs(q[:, :, D:], pos, m["rot"]["base"], m["rot"]["dims"])
    k = (c @ w[p + "uk"].T).view(n, H, D)
    v = (c @ w[p + "uv"].T).view(n, H, V)
    out = torch.zeros(n, H, V, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :D] @ k[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        for i in range(n):
            e = torch.exp(s[i, :i + 1])
            den = e.sum() + torch.exp(w[p + "sink"][hd])
            out[i, hd] = (e / den) @ v[:i + 1, hd]
    return out.reshape(n, H * V) @ w[p + "o"].T


def window_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float) -> torch.Tensor:
    """Grouped-query attention without rotation: unit-RMS values, a logarithmic distance penalty, a sliding window and an
    element-wise sigmoid gate on the heads' outputs."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    win = int(m["mask"]["size"])
    q = (h @ w[p + "q"].T).view(n, H, D)
    k = (h @ w[p + "k"].T).view(n, G, D)
    v = rms_unit((h @ w[p + "v"].T).view(n, G, V), eps)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    out = torch.zeros(n, H, V, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        r1, r2 = w[p + "r1"][hd], w[p + "r2"][hd]
        for i in range(n):
            lo = max(0, i - win + 1)
            js = torch.arange(lo, i + 1)
            s = (k[lo:i + 1, g] @ q[i, hd]) * m["scale"] - r1 * torch.log(1.0 + r2 * (i - js).to(F64))
            pr = torch.softmax(s, 0)
            out[i, hd] = pr @ v[lo:i + 1, g]
    return (out.reshape(n, H * V) * gate) @ w[p + "o"].T


def gla(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float,
        state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gated linear attention, token by token: S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t."""
    n = h.shape[0]
    H, D, V, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = (h @ w[p + "q"].T).view(n, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(n, H, D)
    v = (h @ w[p + "v"].T).view(n, H, V)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(n, H, D)
    S = torch.zeros(H, D, V, dtype=F64) if state is None else state.clone()
    o = torch.zeros(n, H, V, dtype=F64)
    for t in range(n):
        S = alpha[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    y = norm_plain(o, w[p + "norm"], eps).reshape(n, H * V) * silu(h @ w[p + "g"].T)
    return y @ w[p + "o"].T, S


def gated_unit(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(scores: torch.Tensor, top: int, n_groups: int, keep: int) -> List[int]:
    """The experts one token uses: the `top` largest scores among the experts of the `keep` groups whose two largest
    scores sum highest."""
    E = scores.numel()
    size = E // n_groups
    gs = []
    for g in range(n_groups):
        part = sorted(scores[g * size:(g + 1) * size].tolist(), reverse=True)
        gs.append(sum(part[:2]))
    best = sorted(range(n_groups), key=lambda g: (-gs[g], g))[:keep]
    allowed = [e for e in range(E) if e // size in best]
    return sorted(allowed, key=lambda e: (-float(scores[e]), e))[:top]


def moe(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, e: Dict[str, Any]) -> torch.Tensor:
    r = e["router"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for x in route(s[t], int(r["top"]), int(groups["count"]), int(groups["keep"])):
            out[t] += s[t, x] * gated_unit(h[t:t + 1], w, f"{p}e{x}.")[0]
    if e.get("shared"):
        out = out + gated_unit(h, w, p + "shared.")
    return out


def forward(cfg: Dict[str, Any], w: Dict[str, torch.Tensor], tokens: List[int]):
    """Logits [n, vocab] and the stream after every layer [L, n, W] for one whole sequence."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = embedding(tokens, w)
    stack, after = [x], []
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        hin = norm_centered(x, w[p + "norm1"], eps)
        if l["type"] == "latent_attention":
            y = latent_attention(hin, w, p + "mix.", l["mixer"], eps)
        elif l["type"] == "attention":
            y = window_attention(hin, w, p + "mix.", l["mixer"], eps)
        else:
            y, _ = gla(hin, w, p + "mix.", l["mixer"], eps)
        x = x + mult * norm_centered(y, w[p + "norm1b"], eps)
        if l.get("mlp"):
            hin = norm_centered(x, w[p + "norm2"], eps)
            y = gated_unit(hin, w, p + "mlp.") if l["mlp"]["kind"] == "dense" else moe(hin, w, p + "mlp.", l["mlp"])
            x = x + mult * norm_centered(y, w[p + "norm2b"], eps)
        stack.append(x)
        x = sum(w[p + "dwa"][j] * stack[j] for j in range(i + 2))
        after.append(x)
    return norm_centered(x, w["final.norm"], eps) @ w["head"].T, torch.stack(after)


def greedy(cfg: Dict[str, Any], w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """Greedy continuation, recomputing the whole sequence for every new token."""
    toks, out = list(prompt), []
    for _ in range(n_new):
        logits, _ = forward(cfg, w, toks)
        out.append(int(torch.argmax(logits[-1])))
        toks.append(out[-1])
    return out
