"""Parallel blocks on an fp32 residual stream: both sublayers of a layer read one RMS norm of the stream and their
outputs are added to it together.

    h = x / sqrt(mean(x^2) + eps) * w;     x <- x + a(h) + b(h)

GPU: ``csrc/hip/parallel_block.hip``. CPU: PyTorch formulations of the same arithmetic (fp32).
"""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib as L


def embed_scaled(tokens: torch.Tensor, embed: torch.Tensor, scale: float) -> torch.Tensor:
    """tokens int64 [T] -> fp32 stream [T, W] = embed[token] * scale."""
    T, W = tokens.numel(), embed.shape[1]
    if L.use_hip(embed):
        assert tokens.dtype == torch.int64 and embed.is_contiguous()
        out = torch.empty(T, W, dtype=torch.float32, device=embed.device)
        L.check(L.lib().areal_embed_scale(L.ptr(tokens), L.ptr(embed), L.ptr(out), L.c_int(T), L.c_int(W),
                                          L.c_int(embed.shape[0]), L.c_float(scale), L.c_int(L.dtype_flag(embed)),
                                          L.stream_ptr()), "embed_scale")
        return out
    return embed[tokens].float() * float(scale)


def sum_norm(x: torch.Tensor, y1: Optional[torch.Tensor], y2: Optional[torch.Tensor], weight: Optional[torch.Tensor],
             eps: float, dtype: torch.dtype, want32: bool = False
             ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """x fp32 [T, W] <- x + y1 + y2 in place (y's in the compute dtype, None: left out; y2 needs y1). With `weight` the
    RMS norm of the new x is produced by the same launch. Returns (x, norm in fp32 or None unless `want32` / the
    compute dtype is fp32, norm in the compute dtype)."""
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()
    assert y2 is None or y1 is not None
    T, W = x.shape
    if L.use_hip(x):
        for y in (y1, y2):
            assert y is None or (y.dtype == dtype and y.is_contiguous() and y.shape == x.shape)
        assert weight is None or (weight.dtype == dtype and weight.numel() == W)
        f32 = dtype == torch.float32
        o32 = oc = None
        if weight is not None:
            o32 = torch.empty_like(x) if (want32 or f32) else None
            oc = o32 if f32 else torch.empty(T, W, dtype=dtype, device=x.device)
        L.check(L.lib().areal_sum_norm(L.ptr(x), L.ptr(y1), L.ptr(y2), L.ptr(weight), L.ptr(o32),
                                       None if (f32 or oc is None) else L.ptr(oc), L.c_int(T), L.c_int(W),
                                       L.c_float(eps), L.c_int(L.dtype_flag(weight if weight is not None else y1)),
                                       L.stream_ptr()), "sum_norm")
        return x, o32, oc
    if y1 is not None:
        x.add_(y1.float() + y2.float() if y2 is not None else y1.float())
    if weight is None:
        return x, None, None
    h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    return x, h, (h if dtype == torch.float32 else h.to(dtype))


def glu_rows(gu: torch.Tensor, act: str = "silu") -> torch.Tensor:
    """gu [n, 2F] = gate | up (a view with unit stride along the columns) -> act(gate) * up, [n, F] contiguous in gu's
    dtype (fp32 arithmetic); `act` is "silu" or "gelu_tanh"."""
    n, F2 = gu.shape
    Fh = F2 // 2
    if L.use_hip(gu):
        assert gu.stride(1) == 1
        out = torch.empty(n, Fh, dtype=gu.dtype, device=gu.device)
        L.check(L.lib().areal_glu_rows(L.ptr(gu), L.c_int64(gu.stride(0)), L.ptr(out), L.c_int64(n), L.c_int(Fh),
                                       L.c_int(0 if act == "silu" else 1), L.c_int(L.dtype_flag(gu)), L.stream_ptr()),
                "glu_rows")
        return out
    g, u = gu[:, :Fh].float(), gu[:, Fh:].float()
    a = F.silu(g) if act == "silu" else F.gelu(g, approximate="tanh")
    return (a * u).to(gu.dtype)


def relu2_rows(z: torch.Tensor) -> torch.Tensor:
    """max(z, 0)^2 of z [n, F] (a view with unit stride along the columns), contiguous in z's dtype."""
    n, Fh = z.shape
    if L.use_hip(z):
        assert z.stride(1) == 1
        out = torch.empty(n, Fh, dtype=z.dtype, device=z.device)
        L.check(L.lib().areal_relu2_rows(L.ptr(z), L.c_int64(z.stride(0)), L.ptr(out), L.c_int64(n), L.c_int(Fh),
                                         L.c_int(L.dtype_flag(z)), L.stream_ptr()), "relu2_rows")
        return out
    return torch.relu(z.float()).pow(2).to(z.dtype)


ROUTER_KERNEL_MAX_ROWS = 256


def router_logits(h32: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """z = h32 W^T + b in fp32: h32 fp32 [T, W] (a norm's fp32 output), weight [E, W] and bias [E] in the model's
    dtype (read as they are, products and sums in fp32). Few rows (decoding) run one wave per (row, expert); many rows
    the fp32 library product."""
    T, W = h32.shape
    E = weight.shape[0]
    assert h32.dtype == torch.float32
    if L.use_hip(h32) and T <= ROUTER_KERNEL_MAX_ROWS:
        assert h32.is_contiguous() and weight.is_contiguous() and weight.shape == (E, W)
        assert bias is None or (bias.dtype == weight.dtype and bias.numel() == E)
        z = torch.empty(T, E, dtype=torch.float32, device=h32.device)
        L.check(L.lib().areal_router_logits(L.ptr(h32), L.ptr(weight), L.ptr(bias), L.ptr(z), L.c_int(T), L.c_int(W),
                                            L.c_int(E), L.c_int(L.dtype_flag(weight)), L.stream_ptr()), "router_logits")
        return z
    return F.linear(h32, weight.float(), bias.float() if bias is not None else None)
