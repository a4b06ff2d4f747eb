"""Attention through a shared low-rank latent, over a paged cache that holds only the latent and one rotated key.

Per token the cache row is [c | r]: the RMS-normalised latent c (R numbers) and a rotary key part r (P numbers) that
all heads share. Head h has an unrotated key W_uk[h] c and a value W_uv[h] c; neither is ever materialised:

    score_h(i, j) = scale * (q~_h(i) . c(j) + rot(q^r_h(i)) . r(j)),   q~_h = W_uk[h]^T q^n_h     ("absorbed" query)
    o~_h(i)       = sum_j softmax_j(score_h(i, .)) c(j)                 visible: 0 <= i - j < window (<= 0: causal)
    o_h(i)        = W_uv[h] o~_h(i)  [* sigmoid(gate_h(i))]

so the kernel is multi-query attention with key size R + P and value = the first R key entries: a key tile is staged
once and serves both products for every head. The two small per-head products (q~ and o) are batched matrix products
outside the kernel.

Rotation: "rotate half" pairs (i, i + P/2), angle p * base^(-2i/P); cosines and sines come from a table computed in
double precision (`rotary_table`). With `neighbours` the pairs are the projection's columns (2i, 2i + 1) instead; the
rotated pair members are then kept in the order first members | second members, in the cache and in the scored query
alike (a dot product does not see a permutation applied to both sides).

`sink` [H]: one logit per head whose exponential counts once in the softmax denominator; it has no key and no value.

GPU: ``csrc/hip/latent_attn.hip`` (one kernel for prompt portions and, with a split key range, for decoding).
CPU: PyTorch formulations of the same arithmetic (fp32).

Cache layout: [pages, 32, R + P], token-major.
"""
import os
from typing import Optional, Tuple

import torch

from . import _lib as L
from .attention import PAGE_SIZE


DECODE_WORKGROUPS = int(os.environ.get("AREAL_LATENT_DECODE_WORKGROUPS", "256"))


def alloc_latent_cache(num_pages: int, rank: int, rot: int, dtype, device) -> torch.Tensor:
    return torch.zeros(num_pages, PAGE_SIZE, rank + rot, dtype=dtype, device=device)


def rotary_table(base: float, dims: int, n_pos: int, device) -> torch.Tensor:
    """fp32 [n_pos, dims]: cos(p f_i) for i < dims/2, then sin(p f_i); f_i = base^(-2i/dims)."""
    assert dims % 2 == 0
    i = torch.arange(dims // 2, dtype=torch.float64)
    a = torch.arange(n_pos, dtype=torch.float64).unsqueeze(1) * torch.pow(torch.tensor(float(base), dtype=torch.float64),
                                                                          -2.0 * i / dims)
    return torch.cat([a.cos(), a.sin()], 1).float().to(device)


def _rotate(x: torch.Tensor, pos: torch.Tensor, table: torch.Tensor, neighbours: bool = False) -> torch.Tensor:
    """x fp32 [T, ..., P], pos [T] -> rotated (first pair members, then second members)."""
    P = x.shape[-1]
    cs = table[pos.long()]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (P // 2,)
    c, s = cs[:, :P // 2].reshape(shape), cs[:, P // 2:].reshape(shape)
    u, v = (x[..., 0::2], x[..., 1::2]) if neighbours else (x[..., :P // 2], x[..., P // 2:])
    return torch.cat([u * c - v * s, v * c + u * s], -1)


def latent_prep(proj: torch.Tensor, q_rank: int, rank: int, rot: int, q_weight: torch.Tensor, c_weight: torch.Tensor,
                positions: torch.Tensor, slots: torch.Tensor, cache: torch.Tensor, table: torch.Tensor, eps: float,
                neighbours: bool = False) -> torch.Tensor:
    """proj [T, >= q_rank + rank + rot]: query latent | key/value latent | rotary key part (more columns may follow).
    RMS-normalises the two latents (times their weights), rotates the key part at the token's position, writes
    [c | r] of tokens with slot >= 0 into the cache and returns the normalised query latent [T, q_rank] (q_rank may
    be 0: designs whose queries do not pass through a latent; q_weight is then not read)."""
    T = proj.shape[0]
    assert proj.stride(1) == 1 and proj.shape[1] >= q_rank + rank + rot and cache.shape[2] == rank + rot
    assert table.shape[1] == rot and table.dtype == torch.float32
    cq = torch.empty(T, q_rank, dtype=proj.dtype, device=proj.device)
    if L.use_hip(proj):
        assert slots.dtype == torch.int64 and positions.dtype == torch.int32 and cache.dtype == proj.dtype
        assert (q_rank == 0 or q_weight.dtype == proj.dtype) and c_weight.dtype == proj.dtype
        assert table.is_contiguous()
        L.check(L.lib().areal_latent_prep(
            L.ptr(proj), L.c_int64(proj.stride(0)), L.ptr(q_weight), L.ptr(c_weight), L.ptr(positions), L.ptr(slots),
            L.ptr(table), L.c_int(table.shape[0]), L.ptr(cq), L.ptr(cache), L.c_int(T), L.c_int(q_rank), L.c_int(rank),
            L.c_int(rot), L.c_float(eps), L.c_int(int(neighbours)), L.c_int(L.dtype_flag(proj)), L.stream_ptr()),
                "latent_prep")
        return cq
    p = proj.float()
    a, c = p[:, :q_rank], p[:, q_rank:q_rank + rank]
    if q_rank:
        a = a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + eps) * q_weight.float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * c_weight.float()
    r = _rotate(p[:, q_rank + rank:q_rank + rank + rot], positions, table, neighbours)
    cq.copy_(a)
    ok = slots >= 0
    if ok.any():
        pg, off = (slots[ok] // PAGE_SIZE).long(), (slots[ok] % PAGE_SIZE).long()
        cache[pg, off] = torch.cat([c, r], 1)[ok].to(cache.dtype)
    return cq


def decode_splits(batch: int, window: int, max_context: int, heads: int = 16) -> int:
    """Key-range splits of a decode launch: about `DECODE_WORKGROUPS` workgroups (one per row, group of 16 heads and
    split), down to one page each."""
    span = max_context if window <= 0 else min(window + PAGE_SIZE, max_context)
    pages = max(1, (span + PAGE_SIZE - 1) // PAGE_SIZE)
    groups = max(1, batch) * ((heads + 15) // 16)
    return int(max(1, min(DECODE_WORKGROUPS // groups, pages, 32)))


def latent_attention(q: torch.Tensor, q_lat: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor,
                     cu_q: torch.Tensor, ctx_len: torch.Tensor, max_q: int, dim: int, rot: int, scale: float,
                     window: int, table: torch.Tensor, gate: Optional[torch.Tensor] = None, nsplit: int = 1,
                     workspace: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                     matrix_cores: bool = True, neighbours: bool = False,
                     sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, H, dim + rot] (a view whose heads are contiguous; its last `rot` entries per head are the UNROTATED rotary
    query part; the kernel rotates them at the query's position), q_lat [T, H, R] absorbed queries. Row b owns tokens cu_q[b]:cu_q[b+1], the LAST
    positions of its context of ctx_len[b] tokens, whose cache rows are written already. gate [T, H] (unit stride
    along the heads) or None. `matrix_cores`: bf16 rows of several queries with the common latent / rotary sizes run
    the MFMA kernel (False: always the plain one). Returns o~ [T, H, R] (times sigmoid(gate))."""
    T, H, R = q_lat.shape
    B = cu_q.numel() - 1
    assert q.shape == (T, H, dim + rot) and cache.shape[2] == R + rot and table.shape[1] == rot
    if L.use_hip(q):
        assert q.stride(2) == 1 and q.stride(1) == dim + rot and q_lat.is_contiguous()
        assert cache.dtype == q.dtype and q_lat.dtype == q.dtype
        assert sink is None or (sink.dtype == q.dtype and sink.numel() == H and sink.is_contiguous())
        assert block_tables.dtype == torch.int32 and block_tables.is_contiguous()
        assert cu_q.dtype == torch.int32 and ctx_len.dtype == torch.int32
        assert gate is None or (gate.dtype == q.dtype and gate.stride(1) == 1 and gate.shape == (T, H))
        out = torch.empty(T, H, R, dtype=q.dtype, device=q.device)
        pa = pm = None
        if nsplit > 1:
            assert max_q == 1, "split key ranges are for single-query rows"
            if workspace is None:
                workspace = (torch.empty(T * nsplit * H * R, dtype=torch.float32, device=q.device),
                             torch.empty(T * nsplit * H * 2, dtype=torch.float32, device=q.device))
            pa, pm = workspace
            assert pa.numel() >= T * nsplit * H * R and pm.numel() >= T * nsplit * H * 2
        L.check(L.lib().areal_latent_attn(
            L.ptr(q), L.c_int64(q.stride(0)), L.ptr(q_lat), L.ptr(cache), L.ptr(block_tables),
            L.c_int(block_tables.shape[1]), L.ptr(cu_q), L.ptr(ctx_len), L.ptr(table), L.c_int(table.shape[0]),
            L.c_int(int(neighbours)), L.ptr(sink), L.ptr(gate),
            L.c_int64(gate.stride(0) if gate is not None else 0), L.ptr(out), L.ptr(pa), L.ptr(pm), L.c_int(B),
            L.c_int(int(max_q)), L.c_int(T), L.c_int(H), L.c_int(dim), L.c_int(rot), L.c_int(R), L.c_float(scale),
            L.c_int(int(window)), L.c_int(int(nsplit)), L.c_int(L.dtype_flag(q)), L.c_int(int(matrix_cores)),
            L.stream_ptr()), "latent_attn")
        return out
    out = torch.zeros(T, H, R, dtype=torch.float32, device=q.device)
    cq, cl = cu_q.tolist(), ctx_len.tolist()
    for b in range(B):
        n, ctx = cq[b + 1] - cq[b], cl[b]
        if n <= 0:
            continue
        lo = 0 if window <= 0 else max(0, ctx - n - window + 1)
        pages = block_tables[b, :(ctx + PAGE_SIZE - 1) // PAGE_SIZE].long()
        kk = cache[pages].reshape(-1, R + rot)[lo:ctx].float()
        pos = torch.arange(ctx - n, ctx, device=q.device)
        qr = _rotate(q[cq[b]:cq[b + 1], :, dim:].float(), pos, table, neighbours)
        s = (torch.einsum("ihr,jr->hij", q_lat[cq[b]:cq[b + 1]].float(), kk[:, :R])
             + torch.einsum("ihp,jp->hij", qr, kk[:, R:])) * scale
        i = pos.view(n, 1)
        j = torch.arange(lo, ctx, device=q.device).view(1, -1)
        ok = (i - j >= 0) & ((i - j < window) if window > 0 else True)
        s = s.masked_fill(~ok, float("-inf"))
        if sink is not None:  # one more column: the sink's logit, with a zero value
            s = torch.cat([s, sink.float().view(H, 1, 1).expand(H, n, 1)], -1)
        p = torch.softmax(s, -1)[..., :kk.shape[0]]
        out[cq[b]:cq[b + 1]] = torch.einsum("hij,jr->ihr", p, kk[:, :R])
    if gate is not None:
        out = out * torch.sigmoid(gate.float()).unsqueeze(-1)
    return out.to(q.dtype)
