"""Sliding-window attention over the paged cache with shaped scores: soft cap, linear distance bias, mixing of the
heads' scores ahead of the softmax, an optional value-less sink in the denominator, optionally the first tokens of a
sequence kept visible beyond the window. Two ways of preparing queries and keys: RMS norm with a weight
(`qk_norm_cache_write`), or rotation by position followed by a weightless RMS norm, with the values optionally mixed
with those of another layer (`rot_norm_cache_write`).

GPU: ``csrc/hip/window_attn.hip`` (one kernel for prompt portions and, with a split key range, for decoding).
CPU: a PyTorch formulation used by the unit tests and CPU runs.

Cache layout: K [pages, G, 32, D], V [pages, G, 32, Dv] (token-major pages; key and value sizes may differ).
"""
import dataclasses
import math
from typing import Optional, Tuple

import torch

from . import _lib as L
from .attention import PAGE_SIZE


@dataclasses.dataclass
class ScoreShape:
    """Constants of the score pipeline (see the module docstring)."""
    scale: float
    softcap: float = 0.0  # <= 0: no cap
    slope_exp: float = 0.0  # slope of head h: 2^(-slope_exp (h + 1) / H); 0: no distance bias
    window: int = 0  # <= 0: all earlier tokens
    sink: bool = False
    keep_first: int = 0  # keys at positions below this stay visible to every later query, whatever the window


def alloc_window_cache(num_pages: int, n_kv_heads: int, k_dim: int, v_dim: int, dtype, device
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    return (torch.zeros(num_pages, n_kv_heads, PAGE_SIZE, k_dim, dtype=dtype, device=device),
            torch.zeros(num_pages, n_kv_heads, PAGE_SIZE, v_dim, dtype=dtype, device=device))


def qk_norm_cache_write(proj: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                        slots: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, n_heads: int, eps: float
                        ) -> torch.Tensor:
    """proj [T, >= (H + G) D + G Dv]: q heads | k heads | v heads (more columns may follow). RMS-normalises every q
    and k head over D (times the weight vector, shared by the heads), writes k and v of tokens with slot >= 0 into the
    paged caches and returns the normalised queries [T, H, D]."""
    T = proj.shape[0]
    G, D, V = kcache.shape[1], kcache.shape[3], vcache.shape[3]
    H = n_heads
    assert proj.stride(1) == 1 and proj.shape[1] >= (H + G) * D + G * V
    q = torch.empty(T, H, D, dtype=proj.dtype, device=proj.device)
    if L.use_hip(proj):
        assert slots.dtype == torch.int64 and kcache.dtype == proj.dtype
        L.check(L.lib().areal_qk_norm_cache_write(
            L.ptr(proj), L.c_int64(proj.stride(0)), L.ptr(q_weight), L.ptr(k_weight), L.ptr(slots), L.ptr(q),
            L.ptr(kcache), L.ptr(vcache), L.c_int(T), L.c_int(H), L.c_int(G), L.c_int(D), L.c_int(V), L.c_float(eps),
            L.c_int(L.dtype_flag(proj)), L.stream_ptr()), "qk_norm_cache_write")
        return q
    qk = proj[:, :(H + G) * D].float().view(T, H + G, D)
    qk = qk * torch.rsqrt(qk.pow(2).mean(-1, keepdim=True) + eps)
    qn, kn = qk[:, :H], qk[:, H:]
    if q_weight is not None:
        qn = qn * q_weight.float()
    if k_weight is not None:
        kn = kn * k_weight.float()
    q.copy_(qn)
    ok = slots >= 0
    if ok.any():
        pg, off = (slots[ok] // PAGE_SIZE).long(), (slots[ok] % PAGE_SIZE).long()
        kcache[pg, :, off, :] = kn[ok].to(kcache.dtype)
        vcache[pg, :, off, :] = proj[ok, (H + G) * D:(H + G) * D + G * V].view(-1, G, V).to(vcache.dtype)
    return q


def qkv_vnorm_cache_write(proj: torch.Tensor, slots: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                          n_heads: int, eps: float, v_norm: bool = True, v_transposed: bool = False,
                          copy_q: bool = True) -> torch.Tensor:
    """proj [T, >= (H + G) D + G Dv]: q heads | k heads | v heads (more columns may follow). Queries and keys stay as they
    are; with `v_norm` every value head is divided by its root mean square over Dv (no weight) and is cached so. Writes
    k and v of tokens with slot >= 0 into the paged caches (`v_transposed`: V pages [pages, G, Dv, 32]) and returns the
    queries [T, H, D]: a contiguous copy, or (`copy_q` False) the view of proj that holds them."""
    T = proj.shape[0]
    G, D, V = kcache.shape[1], kcache.shape[3], vcache.shape[2 if v_transposed else 3]
    H = n_heads
    assert proj.stride(1) == 1 and proj.shape[1] >= (H + G) * D + G * V
    q = torch.empty(T, H, D, dtype=proj.dtype, device=proj.device) if copy_q else proj[:, :H * D].view(T, H, D)
    if L.use_hip(proj):
        assert slots.dtype == torch.int64 and kcache.dtype == proj.dtype and vcache.dtype == proj.dtype
        L.check(L.lib().areal_qkv_vnorm_cache_write(
            L.ptr(proj), L.c_int64(proj.stride(0)), L.ptr(slots), L.ptr(q) if copy_q else None, L.ptr(kcache),
            L.ptr(vcache), L.c_int(T), L.c_int(H), L.c_int(G), L.c_int(D), L.c_int(V), L.c_float(eps),
            L.c_int(int(v_norm)), L.c_int(int(v_transposed)), L.c_int(L.dtype_flag(proj)), L.stream_ptr()),
            "qkv_vnorm_cache_write")
        return q
    if copy_q:
        q.copy_(proj[:, :H * D].reshape(T, H, D))
    ok = slots >= 0
    if ok.any():
        pg, off = (slots[ok] // PAGE_SIZE).long(), (slots[ok] % PAGE_SIZE).long()
        v = proj[ok, (H + G) * D:(H + G) * D + G * V].float().view(-1, G, V)
        if v_norm:
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        kcache[pg, :, off, :] = proj[ok, H * D:(H + G) * D].view(-1, G, D)
        if v_transposed:
            vcache[pg, :, :, off] = v.to(vcache.dtype)
        else:
            vcache[pg, :, off, :] = v.to(vcache.dtype)
    return q


def sigmoid_gate_rows(x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """x [T, n] (contiguous) <- x * sigmoid(gate) in place; gate [T, n], a view with unit stride along the columns."""
    T, n = x.shape
    assert x.is_contiguous() and gate.shape == x.shape and gate.stride(1) == 1 and gate.dtype == x.dtype
    if L.use_hip(x):
        L.check(L.lib().areal_sigmoid_gate_rows(L.ptr(x), L.ptr(gate), L.c_int64(gate.stride(0)), L.c_int64(T),
                                                L.c_int(n), L.c_int(L.dtype_flag(x)), L.stream_ptr()),
                "sigmoid_gate_rows")
        return x
    x.copy_((x.float() * torch.sigmoid(gate.float())).to(x.dtype))
    return x


def rotation_table(base: float, dims: int, n_pos: int, device, scaling: Optional[dict] = None) -> torch.Tensor:
    """fp32 [n_pos, dims]: m cos(p f_i) for i < dims/2, then m sin(p f_i), with f_i = base^(-2i/dims).

    `scaling` = {factor, original, fast, slow} stretches the slow pairs for contexts beyond `original` positions (YaRN:
    Peng et al., "YaRN: Efficient Context Window Extension of Large Language Models"): with
    d(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) the frequency is f_i (1 - ramp_i) + f_i ramp_i / factor, and
    m = 0.1 ln(factor) + 1 (1 without scaling). Angles are formed in float64 and rounded once."""
    assert dims % 2 == 0 and dims > 0
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    m = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def d_of(turns: float) -> float:
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

        lo = max(math.floor(d_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(d_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        m = 0.1 * math.log(factor) + 1.0
    a = torch.arange(n_pos, dtype=torch.float64).unsqueeze(1) * f
    return (torch.cat([a.cos(), a.sin()], 1) * m).float().to(device)


def rot_norm_cache_write(proj: torch.Tensor, positions: torch.Tensor, table: Optional[torch.Tensor],
                         slots: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, n_heads: int, eps: float,
                         v_first: Optional[torch.Tensor] = None, lam: Optional[torch.Tensor] = None,
                         v_transposed: bool = False) -> torch.Tensor:
    """proj [T, >= (H + G) D + G Dv]: q heads | k heads | v heads (more columns may follow). Rotates the first
    table.shape[1] coordinates of every q and k head at the token's position (pairs (2i, 2i + 1); `table` as
    `rotation_table` makes it, None: no rotation), divides every head by its root mean square over D, and writes k and
    v of tokens with slot >= 0 into the paged caches; with `v_first` [T, G Dv] (a view with unit column stride) and
    `lam` (one number) the values become (1 - lam) v + lam v_first first. `v_transposed`: the V pages are
    [pages, G, Dv, 32] (`alloc_kv_cache`'s layout) instead of [pages, G, 32, Dv]. Returns the queries [T, H, D]."""
    T = proj.shape[0]
    G, D, V = kcache.shape[1], kcache.shape[3], vcache.shape[2 if v_transposed else 3]
    H = n_heads
    R = 0 if table is None else table.shape[1]
    assert proj.stride(1) == 1 and proj.shape[1] >= (H + G) * D + G * V and R <= D and R % 2 == 0
    assert (v_first is None) == (lam is None)
    q = torch.empty(T, H, D, dtype=proj.dtype, device=proj.device)
    if L.use_hip(proj):
        assert slots.dtype == torch.int64 and kcache.dtype == proj.dtype and positions.dtype == torch.int32
        assert table is None or (table.dtype == torch.float32 and table.is_contiguous())
        assert v_first is None or (v_first.dtype == proj.dtype and v_first.stride(1) == 1
                                   and v_first.shape == (T, G * V) and lam.dtype == proj.dtype and lam.numel() == 1)
        if table is None:  # one row of angle zero
            table = torch.zeros(1, 0, dtype=torch.float32, device=proj.device)
        L.check(L.lib().areal_rot_norm_cache_write(
            L.ptr(proj), L.c_int64(proj.stride(0)), L.ptr(positions), L.ptr(table), L.c_int(table.shape[0]), L.c_int(R),
            L.ptr(slots), L.ptr(v_first), L.c_int64(v_first.stride(0) if v_first is not None else 0), L.ptr(lam),
            L.ptr(q), L.ptr(kcache), L.ptr(vcache), L.c_int(T), L.c_int(H), L.c_int(G), L.c_int(D), L.c_int(V),
            L.c_float(eps), L.c_int(int(v_transposed)), L.c_int(L.dtype_flag(proj)), L.stream_ptr()),
            "rot_norm_cache_write")
        return q
    qk = proj[:, :(H + G) * D].float().view(T, H + G, D)
    if R:
        cs = table[positions.long()]
        c, s = cs[:, :R // 2].unsqueeze(1), cs[:, R // 2:].unsqueeze(1)
        u, w = qk[..., 0:R:2], qk[..., 1:R:2]
        rot = torch.stack([u * c - w * s, w * c + u * s], -1).reshape(T, H + G, R)
        qk = torch.cat([rot, qk[..., R:]], -1)
    qk = qk * torch.rsqrt(qk.pow(2).mean(-1, keepdim=True) + eps)
    q.copy_(qk[:, :H])
    v = proj[:, (H + G) * D:(H + G) * D + G * V].float()
    if v_first is not None:
        lam_f = lam.float().reshape(())
        v = (1.0 - lam_f) * v + lam_f * v_first.float()
    ok = slots >= 0
    if ok.any():
        pg, off = (slots[ok] // PAGE_SIZE).long(), (slots[ok] % PAGE_SIZE).long()
        kcache[pg, :, off, :] = qk[:, H:][ok].to(kcache.dtype)
        if v_transposed:
            vcache[pg, :, :, off] = v[ok].view(-1, G, V).to(vcache.dtype)
        else:
            vcache[pg, :, off, :] = v[ok].view(-1, G, V).to(vcache.dtype)
    return q


def standard_layout_ok(dim: int, vdim: int, dtype, device) -> bool:
    """Whether an attention layer without head mixing, cap, bias or sink can live in the engine's standard cache
    (K [pages, G, 32, 128], V transposed) and run its matrix-core flash / paged-decode kernels (which also want at
    most 16 query heads per key/value head)."""
    return dim == vdim == 128 and dtype == torch.bfloat16 and torch.device(device).type == "cuda"


def window_attention_standard(q: torch.Tensor, kcache: torch.Tensor, vcache_t: torch.Tensor, block_tables: torch.Tensor,
                              cu_q: torch.Tensor, cu_k: torch.Tensor, ctx_len: torch.Tensor, max_q: int,
                              shape: ScoreShape, nsplit: int = 1,
                              workspace: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                              log_bias: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                              gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`window_attention` for layers in the standard cache layout (bf16, head size 128, V pages [pages, G, 128, 32]):
    plain scaled scores behind the window that keeps the first tokens. Prompt portions run the paged flash kernel,
    single-query rows the paged decode kernel (``csrc/hip/flash_attn_paged.hip``, ``csrc/hip/paged_attn.hip``), both
    with the softmax weights at 16 bits of mantissa. cu_k int32 [B + 1]: cumulative context lengths. q may be a view
    whose heads are contiguous. log_bias = (r1, r2), both [H]: r1_h ln(1 + r2_h (i - j)) is taken off the scaled score.
    gate [T, H D] (a view with unit stride along the columns): the output times sigmoid(gate), element by element."""
    T, H, D = q.shape
    G = kcache.shape[1]
    B = cu_q.numel() - 1
    assert L.use_hip(q) and q.dtype == torch.bfloat16 and D == 128 and vcache_t.shape[2] == 128
    assert q.stride(2) == 1 and q.stride(1) == D
    r1 = r2 = None
    if log_bias is not None:
        r1, r2 = log_bias
        assert r1.dtype == q.dtype and r2.dtype == q.dtype and r1.numel() == H and r2.numel() == H
        assert r1.is_contiguous() and r2.is_contiguous()
    assert shape.softcap <= 0 and shape.slope_exp == 0 and not shape.sink
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and ctx_len.dtype == torch.int32
    gstride = 0
    if gate is not None:
        assert gate.dtype == q.dtype and gate.shape == (T, H * D) and gate.stride(1) == 1
        assert gate.stride(0) % 4 == 0 and gate.data_ptr() % 8 == 0
        gstride = gate.stride(0)
    out = torch.empty(T, H, D, dtype=q.dtype, device=q.device)
    if max_q == 1:
        assert T == B
        pa = pm = None
        if nsplit > 1:
            if workspace is None:
                workspace = (torch.empty(T * nsplit * H * D, dtype=torch.float32, device=q.device),
                             torch.empty(T * nsplit * H * 2, dtype=torch.float32, device=q.device))
            pa, pm = workspace
            assert pa.numel() >= T * nsplit * H * D and pm.numel() >= T * nsplit * H * 2
        L.check(L.lib().areal_paged_decode_window(
            L.ptr(q), L.ptr(kcache), L.ptr(vcache_t), L.ptr(block_tables), L.ptr(ctx_len), L.ptr(out), L.ptr(pa),
            L.ptr(pm), L.c_int(B), L.c_int(H), L.c_int(G), L.c_int(D), L.c_int(block_tables.shape[1]),
            L.c_int(int(nsplit)), L.c_float(shape.scale), L.c_int(q.stride(0)), L.c_int(int(shape.window)),
            L.c_int(int(shape.keep_first)), L.ptr(r1), L.ptr(r2), L.ptr(gate), L.c_int64(gstride), L.stream_ptr()),
            "paged_decode_window")
        return out
    assert cu_q.dtype == torch.int32 and cu_k.dtype == torch.int32
    L.check(L.lib().areal_flash_fwd_paged_window(
        L.ptr(q), L.ptr(kcache), L.ptr(vcache_t), L.ptr(block_tables), L.c_int(block_tables.shape[1]), L.ptr(out),
        L.ptr(cu_q), L.ptr(cu_k), L.c_int(B), L.c_int(int(max_q)), L.c_int(T), L.c_int(H), L.c_int(G), L.c_int(D),
        L.c_int64(q.stride(0)), L.c_int64(out.stride(0)), L.c_float(shape.scale), L.c_int(int(shape.window)),
        L.c_int(int(shape.keep_first)), L.ptr(r1), L.ptr(r2), L.ptr(gate), L.c_int64(gstride), L.stream_ptr()),
        "flash_fwd_paged_window")
    return out


def decode_splits(batch: int, window: int, max_context: int, keep_first: int = 0) -> int:
    """Key-range splits of a decode launch: about two workgroups per compute unit, down to one page each (a
    workgroup walks its pages one after the other, so short ranges are what makes a decode step short)."""
    span = max_context if window <= 0 else min(window + PAGE_SIZE + max(0, keep_first), max_context)
    pages = max(1, (span + PAGE_SIZE - 1) // PAGE_SIZE)
    return int(max(1, min(512 // max(1, batch), pages, 32)))


def window_attention(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, block_tables: torch.Tensor,
                     cu_q: torch.Tensor, ctx_len: torch.Tensor, max_q: int, shape: ScoreShape,
                     mix: Optional[torch.Tensor] = None, nsplit: int = 1,
                     workspace: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                     gate: Optional[torch.Tensor] = None, matrix_cores: bool = True,
                     log_bias: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> torch.Tensor:
    """q [T, H, D] (row b owns tokens cu_q[b]:cu_q[b+1], the LAST positions of its context of ctx_len[b] tokens,
    whose keys / values are in the cache already). mix [H, H] or None. gate [T, H] (a view with unit stride along
    the heads) or None: head h of token t is multiplied by sigmoid(gate[t, h]); gate [T, H Dv]: one gate per value
    channel. log_bias = (r1, r2), both [H]: r1_h ln(1 + r2_h (i - j)) is taken off the scaled score. `matrix_cores`: bf16 rows of several
    queries with head sizes 64 / 128, value sizes 32 / 64 / 128 and at most 16 heads (without `mix`: any number that
    splits into groups of whole key/value heads) run the MFMA kernel (False: always the plain one).
    Returns [T, H, Dv]."""
    T, H, D = q.shape
    G, V = kcache.shape[1], vcache.shape[3]
    B = cu_q.numel() - 1
    if L.use_hip(q):
        assert q.is_contiguous() and kcache.dtype == q.dtype and block_tables.dtype == torch.int32
        assert cu_q.dtype == torch.int32 and ctx_len.dtype == torch.int32 and block_tables.is_contiguous()
        assert mix is None or (mix.dtype == q.dtype and mix.is_contiguous() and mix.shape == (H, H))
        assert gate is None or (gate.dtype == q.dtype and gate.stride(1) == 1 and gate.shape in ((T, H), (T, H * V)))
        gate_elem = gate is not None and gate.shape[1] == H * V and V > 1
        r1 = r2 = None
        if log_bias is not None:
            r1, r2 = log_bias
            assert r1.dtype == q.dtype and r2.dtype == q.dtype and r1.numel() == H and r2.numel() == H
            assert r1.is_contiguous() and r2.is_contiguous()
        out = torch.empty(T, H, V, dtype=q.dtype, device=q.device)
        want = 1 if max_q == 1 else 16
        while want > 1 and want // 2 >= max_q:
            want //= 2
        bq = int(L.lib().areal_window_attn_tile(L.c_int(H), L.c_int(G), L.c_int(D), L.c_int(V), L.c_int(want)))
        if bq <= 0:
            raise RuntimeError(f"window attention: {H} heads of size {D} / {V} do not fit the kernel's tile memory")
        pa = pm = None
        if nsplit > 1:
            assert max_q == 1, "split key ranges are for single-query rows"
            if workspace is None:
                workspace = (torch.empty(T, nsplit, H, V, dtype=torch.float32, device=q.device),
                             torch.empty(T, nsplit, H, 2, dtype=torch.float32, device=q.device))
            pa, pm = workspace
            assert pa.numel() >= T * nsplit * H * V and pm.numel() >= T * nsplit * H * 2
        L.check(L.lib().areal_window_attn(
            L.ptr(q), L.ptr(kcache), L.ptr(vcache), L.ptr(block_tables), L.c_int(block_tables.shape[1]), L.ptr(cu_q),
            L.ptr(ctx_len), L.ptr(mix), L.ptr(gate), L.c_int64(gate.stride(0) if gate is not None else 0),
            L.c_int(int(gate_elem)), L.ptr(r1), L.ptr(r2), L.ptr(out),
            L.ptr(pa), L.ptr(pm), L.c_int(B), L.c_int(int(max_q)), L.c_int(T),
            L.c_int(H), L.c_int(G), L.c_int(D), L.c_int(V), L.c_int(bq), L.c_float(shape.scale),
            L.c_float(shape.softcap), L.c_float(shape.slope_exp), L.c_int(int(shape.window)),
            L.c_int(int(shape.keep_first)), L.c_int(int(shape.sink)),
            L.c_int(int(nsplit)), L.c_int(L.dtype_flag(q)), L.c_int(int(matrix_cores)), L.stream_ptr()), "window_attn")
        return out
    out = torch.zeros(T, H, V, dtype=torch.float32, device=q.device)
    cq, cl = cu_q.tolist(), ctx_len.tolist()
    rep = H // G
    slopes = (torch.tensor([2.0 ** (-shape.slope_exp * (h + 1) / H) for h in range(H)], device=q.device)
              if shape.slope_exp != 0 else torch.zeros(H, device=q.device))
    for b in range(B):
        n, ctx = cq[b + 1] - cq[b], cl[b]
        if n == 0:
            continue
        lo = 0 if (shape.window <= 0 or shape.keep_first > 0) else max(0, ctx - n - shape.window + 1)
        pages = block_tables[b, :(ctx + PAGE_SIZE - 1) // PAGE_SIZE].long()
        kk = kcache[pages].permute(1, 0, 2, 3).reshape(G, -1, D)[:, lo:ctx].float().repeat_interleave(rep, 0)
        vv = vcache[pages].permute(1, 0, 2, 3).reshape(G, -1, V)[:, lo:ctx].float().repeat_interleave(rep, 0)
        s = torch.einsum("ihd,hjd->hij", q[cq[b]:cq[b + 1]].float(), kk) * shape.scale
        if shape.softcap > 0:
            s = shape.softcap * torch.tanh(s / shape.softcap)
        i = torch.arange(ctx - n, ctx, device=q.device).view(n, 1)
        j = torch.arange(lo, ctx, device=q.device).view(1, -1)
        s = s - slopes.view(H, 1, 1) * (i - j).float()
        if log_bias is not None:
            s = s - log_bias[0].float().view(H, 1, 1) * torch.log1p(log_bias[1].float().view(H, 1, 1)
                                                                      * (i - j).clamp(min=0).float())
        if mix is not None:
            s = torch.einsum("hg,gij->hij", mix.float(), s)
        ok = (i - j >= 0) & (((i - j < shape.window) | (j < shape.keep_first)) if shape.window > 0 else True)
        s = s.masked_fill(~ok, float("-inf"))
        m = s.max(-1, keepdim=True).values
        if shape.sink:
            m = m.clamp(min=0.0)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True) + (torch.exp(-m) if shape.sink else 0.0)
        out[cq[b]:cq[b + 1]] = torch.einsum("hij,hjv->ihv", e / den, vv)
    if gate is not None:
        g = torch.sigmoid(gate.float())
        out = out * (g.view(T, H, V) if gate.shape[1] == H * V and V > 1 else g.unsqueeze(-1))
    return out.to(q.dtype)
