"""Sublayers between two RMS norms on an fp32 residual stream, with a learned average over the network's depth:

    x  <- x + mult * y / sqrt(mean(y^2) + eps) * (off + wb)        y: a sublayer's output, wb: the norm behind it
    X_n = x;  x <- sum_{j <= n} a[j] X_j                           closing a layer: X_0 .. X_n = the stream ahead of
                                                                   the first layer and behind every layer so far
    h   = x / sqrt(mean(x^2) + eps) * (off + w)                    the norm the next sublayer (or the head) reads

off = 1 when the norms' weights are stored around zero (`centered`), else 0.

GPU: ``csrc/hip/depth_avg.hip`` (the three steps of a row in one launch). CPU: PyTorch formulations (fp32).
"""
from typing import Optional, Tuple

import torch

from . import _lib as L


def embed_pos_norm(tokens: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor,
                   pos_table: Optional[torch.Tensor], weight: Optional[torch.Tensor], eps: float, dtype: torch.dtype,
                   x_out: torch.Tensor, centered: bool = True, want32: bool = False
                   ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """x_out fp32 [T, W] <- embed[token] + pos_table[position] (a learned vector per position; None: none). With
    `weight` the norm of it is returned as (fp32 or None unless `want32` / the compute dtype is fp32, compute dtype)."""
    T, W = tokens.numel(), embed.shape[1]
    assert x_out.dtype == torch.float32 and x_out.shape == (T, W) and x_out.is_contiguous()
    f32 = dtype == torch.float32
    if L.use_hip(embed):
        assert tokens.dtype == torch.int64 and positions.dtype == torch.int32 and embed.is_contiguous()
        assert pos_table is None or (pos_table.is_contiguous() and pos_table.dtype == embed.dtype
                                     and pos_table.shape[1] == W)
        o32 = oc = None
        if weight is not None:
            assert weight.dtype == embed.dtype and weight.numel() == W
            o32 = torch.empty(T, W, dtype=torch.float32, device=embed.device) if (want32 or f32) else None
            oc = o32 if f32 else torch.empty(T, W, dtype=dtype, device=embed.device)
        L.check(L.lib().areal_embed_pos_norm(
            L.ptr(tokens), L.ptr(positions), L.ptr(embed), L.ptr(pos_table), L.c_int(embed.shape[0]),
            L.c_int(pos_table.shape[0] if pos_table is not None else 0), L.ptr(weight), L.ptr(x_out), L.ptr(o32),
            None if (f32 or oc is None) else L.ptr(oc), L.c_int(T), L.c_int(W), L.c_float(eps), L.c_int(int(centered)),
            L.c_int(L.dtype_flag(embed)), L.stream_ptr()), "embed_pos_norm")
        return o32, oc
    x = embed[tokens.clamp(0, embed.shape[0] - 1)].float()
    if pos_table is not None:
        x = x + pos_table[positions.long().clamp(0, pos_table.shape[0] - 1)].float()
    x_out.copy_(x)
    if weight is None:
        return None, None
    h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (weight.float() + (1.0 if centered else 0.0))
    return h, (h if f32 else h.to(dtype))


def norm_add_avg_norm(x: torch.Tensor, y: Optional[torch.Tensor], wb: Optional[torch.Tensor], mult: float,
                      stack: Optional[torch.Tensor], n_stack: int, avg: Optional[torch.Tensor],
                      w_next: Optional[torch.Tensor], eps: float, dtype: torch.dtype, centered: bool = True,
                      want32: bool = False, out: Optional[torch.Tensor] = None
                      ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """x fp32 [T, W]: the stream. With `y` (compute dtype) x + mult * norm_wb(y) is formed and stored in `out` (fp32
    [T, W]; None: in x itself). With `stack` (fp32 [>= n_stack, T, W], n_stack >= 1) the new stream is stored as
    stack[n_stack - 1] (which `out`, when given, has to be) and the stream that goes on is sum_j avg[j] stack[j] over
    j < n_stack. With `w_next` the norm of the stream that goes on is produced by the same launch. Returns (the stream that goes on, its norm in fp32 or None unless `want32` / the
    compute dtype is fp32, its norm in the compute dtype)."""
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()
    T, W = x.shape
    f32 = dtype == torch.float32
    averaged = stack is not None and n_stack > 0
    if averaged:
        assert stack.dtype == torch.float32 and stack.is_contiguous() and stack.shape[1:] == (T, W)
        assert n_stack <= stack.shape[0] and avg is not None and avg.numel() == n_stack
        assert out is None or out.data_ptr() == stack[n_stack - 1].data_ptr()
        out = stack[n_stack - 1]
    elif out is None:
        out = x
    assert out.dtype == torch.float32 and out.shape == x.shape and out.is_contiguous()
    if L.use_hip(x):
        assert y is None or (y.dtype == dtype and y.is_contiguous() and y.shape == x.shape and wb.dtype == dtype)
        assert w_next is None or (w_next.dtype == dtype and w_next.numel() == W)
        assert avg is None or (avg.dtype == dtype and avg.is_contiguous())
        o32 = oc = None
        if w_next is not None:
            o32 = torch.empty_like(x) if (want32 or f32) else None
            oc = o32 if f32 else torch.empty(T, W, dtype=dtype, device=x.device)
        mix = torch.empty_like(x) if averaged else None
        x_out = out if (averaged or y is not None or out.data_ptr() != x.data_ptr()) else None
        some = w_next if w_next is not None else (wb if wb is not None else avg)
        L.check(L.lib().areal_norm_add_avg_norm(
            L.ptr(x), L.ptr(x_out), L.ptr(y), L.ptr(wb), L.c_float(mult), L.ptr(stack) if averaged else None,
            L.c_int64(T * W), L.c_int(n_stack if averaged else 0), L.ptr(avg) if averaged else None, L.ptr(mix),
            L.ptr(w_next), L.ptr(o32), None if (f32 or oc is None) else L.ptr(oc), L.c_int(T), L.c_int(W),
            L.c_float(eps), L.c_int(int(centered)), L.c_int(L.dtype_flag(some)), L.stream_ptr()), "norm_add_avg_norm")
        return (mix if averaged else out), o32, oc
    off = 1.0 if centered else 0.0
    if y is not None:
        yf = y.float()
        out.copy_(x + mult * (yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * (wb.float() + off)))
    elif out.data_ptr() != x.data_ptr():
        out.copy_(x)
    x = out
    if averaged:
        x = (stack[:n_stack] * avg.float().view(n_stack, 1, 1)).sum(0)
    if w_next is None:
        return x, None, None
    h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (w_next.float() + off)
    return x, h, (h if f32 else h.to(dtype))
