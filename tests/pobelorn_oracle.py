"""Plain float64 formulation of the Pobelorn design, one function per mechanism, written from its equations with
loops over tokens where that is the clearest form. It shares no code with the package: the tests compare the
package's ops, model runner and engine against it.

A model is (config dict as in config.json, {tensor name: tensor}); layers are parallel blocks

    h = rms(x) * w1;   x <- x + mixer(h) + ff(h)

with an `attention` mixer (rotated, unit-RMS queries and keys, sliding window that keeps the first tokens, values
mixed with those of the first such layer) or a `lightning` mixer (linear attention with a fixed decay per head), and a
dense squared-ReLU or routed + shared gated feed-forward.
"""
import math
from typing import Dict, List, Optional, Tuple

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotation_frequencies(rot: Dict) -> Tuple[torch.Tensor, float]:
    """Angular frequency of every rotated pair and the factor on cosines and sines."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):  # the (fractional) pair index whose wavelength fits `turns` times into the original length
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(float(f[i]) / factor * ramp + float(f[i]) * (1 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, pos: int, rot: Dict) -> torch.Tensor:
    """x [heads, dim] of the token at position `pos`: neighbouring coordinates (2i, 2i + 1) below rot.dims turn."""
    f, m = rotation_frequencies(rot)
    y = x.clone()
    for i in range(int(rot["dims"]) // 2):
        a = pos * float(f[i])
        c, s = math.cos(a) * m, math.sin(a) * m
        u, v = x[:, 2 * i], x[:, 2 * i + 1]
        y[:, 2 * i] = u * c - v * s
        y[:, 2 * i + 1] = v * c + u * s
    return y


def visible(i: int, j: int, mask: Optional[Dict]) -> bool:
    if j > i:
        return False
    if not mask or not mask.get("size"):
        return True
    return i - j < int(mask["size"]) or j < int(mask.get("keep_first") or 0)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float,
                    v_first: Optional[torch.Tensor], pos0: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """h [n, width] of one sequence (positions pos0 ..) -> (mixer output [n, width], the values that were attended
    [n, G, vdim]). `v_first`: values of the first value-mixing layer, or None when this layer is that one or mixes
    nothing."""
    n = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).view(n, H, D)
    k = (h @ w["k"].T).view(n, G, D)
    v = (h @ w["v"].T).view(n, G, V)
    if m.get("rot"):
        q = torch.stack([rotate(q[t], pos0 + t, m["rot"]) for t in range(n)])
        k = torch.stack([rotate(k[t], pos0 + t, m["rot"]) for t in range(n)])
    q, k = rms(q, eps), rms(k, eps)
    if v_first is not None:
        lam = w["vmix"].to(F64)
        v = (1 - lam) * v + lam * v_first
    out = torch.zeros(n, H, V, dtype=F64)
    for t in range(n):
        js = [j for j in range(t + 1) if visible(pos0 + t, pos0 + j, m.get("mask"))]
        for hd in range(H):
            g = hd // (H // G)
            s = torch.stack([(q[t, hd] * k[j, g]).sum() for j in js]) * float(m["scale"])
            p = torch.softmax(s, 0)
            out[t, hd] = (p.unsqueeze(-1) * torch.stack([v[j, g] for j in js])).sum(0)
    return out.reshape(n, H * V) @ w["o"].T, v


def lightning_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float,
                    state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Linear attention with one decay per head: S <- decay S + k v^T, o = S^T q. Returns (output [n, width], final
    state [H, D, V])."""
    n = h.shape[0]
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    silu = torch.nn.functional.silu
    q = silu(h @ w["q"].T).view(n, H, D)
    k = silu(h @ w["k"].T).view(n, H, D)
    v = silu(h @ w["v"].T).view(n, H, V)
    S = torch.zeros(H, D, V, dtype=F64) if state is None else state.clone()
    o = torch.zeros(n, H, V, dtype=F64)
    for t in range(n):
        for hd in range(H):
            S[hd] = float(m["decay"][hd]) * S[hd] + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    y = rms(o.reshape(n, H * V), eps) * w["norm"]
    y = y * torch.sigmoid(h @ w["g"].T)
    return y @ w["o"].T, S


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return torch.relu(h @ w["up"].T) ** 2 @ w["down"].T


def gated_expert(h: torch.Tensor, gate, up, down) -> torch.Tensor:
    return (torch.nn.functional.silu(h @ gate.T) * (h @ up.T)) @ down.T


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], e: Dict) -> torch.Tensor:
    n = h.shape[0]
    E, top = int(e["router"]["experts"]), int(e["router"]["top"])
    z = h @ w["router"].T + w["router.b"]
    out = torch.zeros_like(h)
    for t in range(n):
        order = sorted(range(E), key=lambda i: -float(z[t, i]))[:top]
        p = torch.softmax(torch.stack([z[t, i] for i in order]), 0)
        for pi, i in zip(p, order):
            out[t] += pi * gated_expert(h[t], w[f"e{i}.gate"], w[f"e{i}.up"], w[f"e{i}.down"])
    if e.get("shared"):
        out = out + gated_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(F64) for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> Tuple[torch.Tensor, List[torch.Tensor]]:
    """One whole sequence -> (logits [n, vocab], the stream after every layer)."""
    eps = float(cfg["norm"]["eps"])
    E = weights["embed"].to(F64)
    x = E[torch.tensor(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    v_first = None
    streams = []
    for i, l in enumerate(cfg["layers"]):
        h = rms(x, eps) * weights[f"l{i}.norm1"].to(F64)
        mw = sub(weights, f"l{i}.mix.")
        if l["type"] == "attention":
            mixing = bool(l["mixer"].get("v_mix"))
            y, v = attention_mixer(h, mw, l["mixer"], eps, v_first if mixing else None)
            if mixing and v_first is None:
                v_first = v
        elif l["type"] == "lightning":
            y, _ = lightning_mixer(h, mw, l["mixer"], eps)
        else:
            raise ValueError(l["type"])
        if l.get("mlp"):
            fw = sub(weights, f"l{i}.mlp.")
            y = y + (dense_ff(h, fw) if l["mlp"]["kind"] == "dense" else moe_ff(h, fw, l["mlp"]))
        x = x + y
        streams.append(x.clone())
    logits = (rms(x, eps) * weights["final.norm"].to(F64)) @ E.T
    return logits, streams


def greedy(cfg: Dict, weights: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n_new):
        logits, _ = forward(cfg, weights, toks)
        out.append(int(torch.argmax(logits[-1])))
        toks.append(out[-1])
    return out
