"""Gated linear attention: a matrix state per head whose rows decay by a data-dependent factor per key channel, carried
as fp32 state per request slot:

    alpha_t = sigmoid(z_t)^(1 / tau)                                  z_t [heads, D]: decay logits
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T (q_t * q_scale)
    y_t = o_t / rms(o_t over V) * w * silu(g_t)                       per head, w [V] shared by the heads

GPU: ``csrc/hip/gla.hip`` (token-by-token scan for decoding and short portions; chunks of 16 tokens for prompt
portions: one launch forms what does not depend on the state for all chunks at once, the next walks the chunks with
matrix products only). CPU: the same recurrence in PyTorch, token by token (fp32).
"""
from typing import Optional

import torch
import torch.nn.functional as F

from . import _lib as L


CHUNK = 16  # tokens per chunk of the chunked form


def alloc_state(n_slots: int, n_heads: int, k_dim: int, v_dim: int, device) -> torch.Tensor:
    """State slots [slots, heads, D, V] fp32. A row that starts at position 0 ignores what its slot held, so slots
    are handed on without clearing."""
    return torch.zeros(n_slots, n_heads, k_dim, v_dim, dtype=torch.float32, device=device)


def gla_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, z: torch.Tensor, z_bias: Optional[torch.Tensor],
             tau: float, q_scale: float, cu_q: torch.Tensor, first_pos: torch.Tensor, state_slots: torch.Tensor,
             state: torch.Tensor, max_q: int = 1) -> torch.Tensor:
    """Advance the state of every row's slot over the row's tokens. proj [T, *] holds heads x D queries at column
    q_off, heads x D keys at k_off, heads x V values at v_off. z fp32 [T, heads D] decay logits (z_bias [heads D] in
    proj's dtype is added, or None). first_pos [B] int32: position of each row's first token (0: fresh state);
    state_slots [B] int32 (negative: the row is skipped). Returns the read-out [T, heads, V] fp32."""
    T = proj.shape[0]
    NH, D, V = state.shape[1], state.shape[2], state.shape[3]
    B = cu_q.numel() - 1
    assert z.dtype == torch.float32 and z.shape == (T, NH * D) and z.stride(1) == 1
    if L.use_hip(proj):
        assert proj.stride(1) == 1 and cu_q.dtype == torch.int32 and first_pos.dtype == torch.int32
        assert state_slots.dtype == torch.int32 and state.dtype == torch.float32 and state.is_contiguous()
        assert min(q_off, k_off, v_off) >= 0 and max(q_off + NH * D, k_off + NH * D, v_off + NH * V) <= proj.shape[1]
        assert z_bias is None or (z_bias.dtype == proj.dtype and z_bias.numel() == NH * D)
        if D > 256:
            raise RuntimeError("gated linear attention: key size above 256 is not built")
        obuf = torch.empty(T, NH, V, dtype=torch.float32, device=proj.device)
        scratch = None
        if max_q >= CHUNK and D <= 128:  # the chunked form's state-independent operands
            scratch = torch.empty(T * (3 * NH * D + CHUNK * NH), dtype=torch.float32, device=proj.device)
        L.check(L.lib().areal_gla_scan(
            L.ptr(proj), L.c_int64(proj.stride(0)), L.c_int(q_off), L.c_int(k_off), L.c_int(v_off), L.ptr(z),
            L.c_int64(z.stride(0)), L.ptr(z_bias), L.c_float(tau), L.c_float(q_scale), L.ptr(cu_q), L.ptr(first_pos),
            L.ptr(state_slots), L.ptr(state), L.ptr(obuf), L.ptr(scratch), L.c_int(T), L.c_int(B), L.c_int(NH),
            L.c_int(D), L.c_int(V),
            L.c_int(int(max_q)), L.c_int(L.dtype_flag(proj)), L.stream_ptr()), "gla_scan")
        return obuf
    obuf = torch.zeros(T, NH, V, dtype=torch.float32, device=proj.device)
    cq, fp, sl = cu_q.tolist(), first_pos.tolist(), state_slots.tolist()
    zz = z + z_bias.float() if z_bias is not None else z
    alpha = torch.exp(F.logsigmoid(zz) / float(tau)).view(T, NH, D)
    for b in range(B):
        if sl[b] < 0 or cq[b + 1] <= cq[b]:
            continue
        S = torch.zeros(NH, D, V) if fp[b] == 0 else state[sl[b]].clone()
        for t in range(cq[b], cq[b + 1]):
            q = proj[t, q_off:q_off + NH * D].float().view(NH, D) * float(q_scale)
            k = proj[t, k_off:k_off + NH * D].float().view(NH, D)
            v = proj[t, v_off:v_off + NH * V].float().view(NH, V)
            S = alpha[t].unsqueeze(2) * S + k.unsqueeze(2) * v.unsqueeze(1)
            obuf[t] = torch.einsum("hdv,hd->hv", S, q)
        state[sl[b]] = S
    return obuf


def gla_out(obuf: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """obuf [T, heads, V] fp32 -> per head o / rms(o over V) * weight * silu(gate) as [T, heads V] in the compute dtype.
    gate: [T, heads V] view with unit stride along the last axis; weight [V]."""
    T, NH, V = obuf.shape
    if L.use_hip(obuf):
        assert obuf.is_contiguous() and gate.stride(1) == 1 and gate.shape == (T, NH * V)
        assert weight.dtype == gate.dtype and weight.numel() == V
        out = torch.empty(T, NH * V, dtype=gate.dtype, device=gate.device)
        L.check(L.lib().areal_gla_out(L.ptr(obuf), L.ptr(gate), L.c_int64(gate.stride(0)), L.ptr(weight), L.ptr(out),
                                      L.c_int(T), L.c_int(NH), L.c_int(V), L.c_float(eps), L.c_int(L.dtype_flag(gate)),
                                      L.stream_ptr()), "gla_out")
        return out
    y = obuf * torch.rsqrt(obuf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    return (y.reshape(T, NH * V) * F.silu(gate.float())).to(gate.dtype)
