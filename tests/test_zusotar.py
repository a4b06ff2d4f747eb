"""Zusotar (layer-list decoder whose sublayers sit between two RMS norms, with a learned average over depth: latent
attention with a sink, window attention with a logarithmic distance penalty on unit-RMS values, gated linear attention,
gated and group-routed feed-forward) against the plain float64 formulation in ``zusotar_oracle.py``: every mechanism
alone, then the serving engine - scheduler, paged caches, state slots, prefill and decode plans - on small random models
of several shapes. Every test runs on the CPU formulations of the ops and, marked `gpu`, on the HIP kernels."""
import math
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import zusotar_oracle as O  # noqa: E402

from areal_vllm_amd.api.cli_args import InferenceServerConfig  # noqa: E402
from areal_vllm_amd.inference.engine import NativeInferenceEngine  # noqa: E402
from areal_vllm_amd.models.config import ModelConfig  # noqa: E402
from areal_vllm_amd.models.hybrid import RoutedSwiGLUExperts  # noqa: E402
from areal_vllm_amd.ops import depth_avg as da  # noqa: E402
from areal_vllm_amd.ops import gla as gla_ops  # noqa: E402
from areal_vllm_amd.ops import latent_attention as lattn  # noqa: E402
from areal_vllm_amd.ops import moe as moe_ops  # noqa: E402
from areal_vllm_amd.ops import window_attention as wattn  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
OP_CASES = [("cpu", torch.float32), ("cpu", torch.bfloat16),
            pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
            pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]
F64 = torch.float64
PAGE = 32


def tol(dtype):
    return 2e-4 if dtype in ("float32", torch.float32) else 6e-2


def row_errors(got, want):
    got, want = torch.as_tensor(got).to(F64), torch.as_tensor(want).to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = (want - want.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().clamp(min=1e-9)
    return d.pow(2).mean(-1).sqrt() / ref


def rel_err(got, want):
    """Per row: rms of the difference (mean taken off) over the rms of the reference row; the largest."""
    return float(row_errors(got, want).max())


def rows_agree(got, want, dtype):
    """32-bit: the median row (of more than two) within the tolerance and every row within ten times it (a head's
    read-out that happens to be close to zero - a first token whose query and key are nearly orthogonal - is blown up
    by the norm behind it, rounding included, and the next tokens read that token). bf16: a router's near-tie may pick another expert for a token (and what reads that token
    shifts with it): the median row must be inside the tolerance and four rows of five within 2.5 times it (a wrong
    kernel is off by the rows' own size; the kernels are held to the sharp bound by the mechanism tests)."""
    e = row_errors(got, want)
    if dtype in ("float32", torch.float32):
        return bool((e.numel() <= 2 or e.median() < tol(dtype)) and e.max() < 10 * tol(dtype))
    return bool(e.median() < tol(dtype) and (e < 2.5 * tol(dtype)).double().mean() >= 0.8)


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


def _slots(pages, lo, hi, device):
    return torch.tensor([pages[p // PAGE] * PAGE + p % PAGE for p in range(lo, hi)], dtype=torch.int64, device=device)


def seen(x, dtype):
    """What the kernels see of a tensor held in `dtype`, as float64."""
    return x.to(dtype).to(F64)


# ------------------------------------------------------------------------------------ mechanisms
@pytest.mark.parametrize("device,dtype", OP_CASES)
def test_embedding_with_positions_closing_sums_and_depth_average(device, dtype):
    g = torch.Generator().manual_seed(3)
    eps = 1e-5
    for T, W in ((5, 48), (3, 257), (1, 8), (2, 1032), (1, 4100), (4, 2048)):
        E, P = torch.randn(19, W, generator=g).to(dtype), torch.randn(11, W, generator=g).to(dtype)
        w1 = (0.2 * torch.randn(W, generator=g)).to(dtype)
        toks, pos = torch.randint(0, 19, (T,), generator=g), torch.randint(0, 11, (T,), generator=g).int()
        n_layers = 3
        stack = torch.full((n_layers + 1, T, W), 77.0, device=device)
        h32, hc = da.embed_pos_norm(toks.to(device), pos.to(device), E.to(device), P.to(device), w1.to(device), eps, dtype,
                                    stack[0], want32=True)
        X = [E.to(F64)[toks] + P.to(F64)[pos.long()]]
        assert rel_err(stack[0].cpu(), X[0]) < 1e-6
        want = O.norm_centered(X[0], w1.to(F64), eps)
        assert h32.dtype == torch.float32 and rel_err(h32.cpu(), want) < 1e-5
        assert hc.dtype == dtype and rel_err(hc.float().cpu(), want) < tol(dtype)
        x = stack[0]
        xw = X[0]
        for li in range(n_layers):
            y1 = (3 * torch.randn(T, W, generator=g)).to(dtype)
            y2 = (0.1 * torch.randn(T, W, generator=g)).to(dtype)
            wb1, wb2, w2, wn = [(0.2 * torch.randn(W, generator=g)).to(dtype) for _ in range(4)]
            avg = torch.randn(li + 2, generator=g).to(dtype)
            # the first closing of a layer: the sum goes to the layer's own slot, the stream it came from stays
            before = x.clone()
            x1, a32, ac = da.norm_add_avg_norm(x, y1.to(device), wb1.to(device), 0.35, None, 0, None, w2.to(device), eps,
                                               dtype, want32=True, out=stack[li + 1])
            xw1 = xw + 0.35 * O.norm_centered(y1.to(F64), wb1.to(F64), eps)
            assert x1.data_ptr() == stack[li + 1].data_ptr() and torch.equal(x, before)
            assert rel_err(x1.cpu(), xw1) < 1e-6 and rel_err(a32.cpu(), O.norm_centered(xw1, w2.to(F64), eps)) < 1e-5
            assert rel_err(ac.float().cpu(), O.norm_centered(xw1, w2.to(F64), eps)) < tol(dtype)
            # the second closing: sum in place, then the average over all streams so far and the next norm
            x2, b32, bc = da.norm_add_avg_norm(x1, y2.to(device), wb2.to(device), 0.35, stack, li + 2, avg.to(device),
                                               wn.to(device) if li + 1 < n_layers else None, eps, dtype, want32=True,
                                               out=stack[li + 1])
            X.append(xw1 + 0.35 * O.norm_centered(y2.to(F64), wb2.to(F64), eps))
            xw = sum(avg.to(F64)[j] * X[j] for j in range(li + 2))
            assert rel_err(stack[li + 1].cpu(), X[-1]) < 1e-6 and rel_err(x2.cpu(), xw) < 2e-6
            if li + 1 < n_layers:
                assert rel_err(b32.cpu(), O.norm_centered(xw, wn.to(F64), eps)) < 1e-5
                assert rel_err(bc.float().cpu(), O.norm_centered(xw, wn.to(F64), eps)) < tol(dtype)
            else:
                assert b32 is None and bc is None
            x = x2
        # the norm alone (ahead of the head), and a layer without a feed-forward: one closing that averages
        _, f32, fc = da.norm_add_avg_norm(x, None, None, 1.0, None, 0, None, w1.to(device), eps, dtype, want32=True)
        assert rel_err(f32.cpu(), O.norm_centered(xw, w1.to(F64), eps)) < 1e-5
        y = torch.randn(T, W, generator=g).to(dtype)
        avg = torch.randn(2, generator=g).to(dtype)
        st2 = torch.zeros(2, T, W, device=device)
        st2[0].copy_(x)
        x3, _, c3 = da.norm_add_avg_norm(st2[0], y.to(device), w1.to(device), 2.0, st2, 2, avg.to(device), w1.to(device),
                                         eps, dtype, out=st2[1])
        new = xw + 2.0 * O.norm_centered(y.to(F64), w1.to(F64), eps)
        mixed = avg.to(F64)[0] * xw + avg.to(F64)[1] * new
        assert rel_err(x3.cpu(), mixed) < 2e-6 and rel_err(c3.float().cpu(), O.norm_centered(mixed, w1.to(F64), eps)) < tol(dtype)


def _paged(n_pages, G, D, V, dtype, device, fill=9.0):
    kc, vc = wattn.alloc_window_cache(n_pages, G, D, V, dtype, device)
    kc.fill_(fill)  # what an earlier request left behind
    vc.fill_(-fill)
    return kc, vc


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("H,G,D,V", [(4, 2, 16, 8), (3, 3, 10, 5), (2, 1, 64, 96), (1, 1, 8, 1), (6, 3, 96, 40)])
def test_unit_rms_values_and_cache_write(device, dtype, H, G, D, V):
    g = torch.Generator().manual_seed(H + D)
    T, lead = 7, 3
    wide = (2 * torch.randn(T, lead + (H + G) * D + G * V + 5, generator=g)).to(dtype)
    proj = wide.to(device)[:, lead:]
    kc, vc = _paged(4, G, D, V, dtype, device)
    slots = torch.tensor([33, 34, -1, 64, 2, 95, 0], dtype=torch.int64, device=device)
    q = wattn.qkv_vnorm_cache_write(proj, slots, kc, vc, H, 1e-5)
    src = wide[:, lead:].to(F64)
    assert q.is_contiguous() and torch.equal(q.cpu().to(F64).reshape(T, -1), src[:, :H * D])
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        pg, off = s // PAGE, s % PAGE
        assert torch.equal(kc[pg, :, off].cpu().to(F64).reshape(-1), src[t, H * D:(H + G) * D])
        want = O.rms_unit(src[t, (H + G) * D:(H + G) * D + G * V].view(G, V), 1e-5)
        assert rel_err(vc[pg, :, off].float().cpu().reshape(1, -1), want.reshape(1, -1)) < tol(dtype)
    assert float(kc[3].float().min()) == 9.0 and float(vc[1, :, 3:].float().max()) == -9.0  # nothing else is touched


def _window_case(H, G, D, V, window, scale, n, probes, seed):
    """Queries, keys, values and gates of one sequence as the columns of an identity-like projection, so that the
    oracle's mixer and the ops see the same numbers. `probes`: (query position, key position) pairs whose score is made
    to stand out: a key just outside the window then shows as a row that is off by its own size."""
    g = torch.Generator().manual_seed(seed)
    width = (H + G) * D + G * V + H * V
    h = torch.randn(n, width, generator=g)
    h[:, H * D:(H + G) * D] *= 0.3
    for qi, kj in probes:
        for c in range(G):
            h[kj, H * D + c * D:H * D + (c + 1) * D] = 3.0 * h[qi, c * (H // G) * D:c * (H // G) * D + D]
    eye = torch.eye(width, dtype=F64)
    a, b, c = H * D, (H + G) * D, (H + G) * D + G * V
    w = {"q": eye[:a], "k": eye[a:b], "v": eye[b:c], "g": eye[c:], "o": torch.eye(H * V, dtype=F64),
         "r1": 0.2 + 0.6 * torch.rand(H, generator=g, dtype=F64), "r2": 0.1 + torch.rand(H, generator=g, dtype=F64)}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale, "mask": {"size": window}}
    return h, w, m


def _run_window(h, w, m, dtype, device, portions, pages, nsplit=1, matrix_cores=True):
    """The ops over a paged cache, the sequence fed in portions; returns [n, H V]."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    kc, vc = _paged(max(pages) + 2, G, D, V, dtype, device, fill=50.0)
    shape = wattn.ScoreShape(scale=m["scale"], window=m["mask"]["size"])
    bt = torch.tensor([pages], dtype=torch.int32, device=device)
    r1, r2 = w["r1"].to(dtype).to(device), w["r2"].to(dtype).to(device)
    outs, at = [], 0
    hd = h.to(dtype).to(device)
    for c in portions:
        c = min(c, n - at)
        if c <= 0:
            break
        rows = hd[at:at + c]
        q = wattn.qkv_vnorm_cache_write(rows, _slots(pages, at, at + c, device), kc, vc, H, 1e-6)
        o = wattn.window_attention(q, kc, vc, bt, i32([0, c], device), i32([at + c], device), c, shape, None,
                                   nsplit=nsplit if c == 1 else 1, matrix_cores=matrix_cores,
                                   gate=rows[:, (H + G) * D + G * V:], log_bias=(r1, r2))
        outs.append(o.reshape(c, H * V).float().cpu())
        at += c
    return torch.cat(outs)


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 16, 8, 37), (2, 1, 8, 8, 32), (3, 3, 12, 20, 5), (1, 1, 16, 4, 64),
                                            (2, 2, 8, 8, 1), (4, 1, 64, 32, 33), (2, 1, 64, 64, 70), (2, 2, 16, 16, 1000),
                                            (6, 2, 128, 128, 41)])
def test_window_edges_distance_penalty_gate_pages_portions_and_splits(device, dtype, H, G, D, V, window):
    n = 150
    w_eff = min(window, n)
    probes = []
    for qi in (n - 1, n - 2, 100, 97, 64, 63, 33, 32, 31):
        probes += [(qi, qi - w_eff + 1), (qi, qi - w_eff)]  # the window's last key, and the first one outside it
        probes += [(qi, 1), (qi, qi - 31), (qi, qi - 32), (qi, qi - 33)]  # far back; around a page's border
    probes = [(a, b) for a, b in probes if 0 <= b <= a]
    for k, (qi, kj) in enumerate(probes):
        h, w, m = _window_case(H, G, D, V, window, 4.0 / math.sqrt(D) * 3, n, [(qi, kj)], 7 + k % 3)
        hs = {key: (seen(val, dtype) if key in ("r1", "r2") else val) for key, val in w.items()}
        want = O.window_attention(seen(h, dtype)[:qi + 1], hs, "", m, 1e-6)
        pages = [3, 1, 4, 9, 2][:(n + PAGE - 1) // PAGE]
        for portions, nsplit in (([n], 1), ([qi, 1, n], 1), ([qi, 1, n], 3), ([max(qi - 1, 1), 2, n], 1)):
            if k % 4 != len(portions) % 4 and portions != [qi, 1, n]:
                continue  # every probe as a decoded token; the other ways of cutting in turn
            got = _run_window(h, w, m, dtype, device, portions, pages, nsplit)
            assert rel_err(got[qi:qi + 1], want[qi:qi + 1]) < tol(dtype), (qi, kj, portions, nsplit)
    # a whole sequence cut in several ways, on both kernels for prompt portions
    h, w, m = _window_case(H, G, D, V, window, 1.0 / math.sqrt(D), n, [], 1)
    hs = {key: (seen(val, dtype) if key in ("r1", "r2") else val) for key, val in w.items()}
    want = O.window_attention(seen(h, dtype), hs, "", m, 1e-6)
    for portions, mc in (([n], True), ([n], False), ([1], True), ([2], True), ([3, 17, 1, 1, 64, 31, 2, 33], True),
                         ([70, 1], True)):
        got = _run_window(h, w, m, dtype, device, portions + [portions[-1]] * n, [6, 0, 3, 8, 1], 2, mc)
        assert rel_err(got, want) < tol(dtype), (portions, mc)
    # the distance penalty is no small correction: without it the rows are off by far more than the tolerance
    if window >= 30:
        flat = dict(hs, r1=torch.zeros(H, dtype=F64))
        assert rel_err(O.window_attention(seen(h, dtype), flat, "", m, 1e-6), want) > 0.1


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,window", [(4, 2, 70), (2, 1, 64), (4, 4, 200), (2, 2, 1000), (3, 1, 1), (16, 1, 33)])
def test_standard_cache_layout_kernels_with_distance_penalty(H, G, window):
    """bf16 heads of 128 live in the engine's standard cache (V pages transposed) and run its paged flash and paged
    decode kernels with the distance penalty: window edges, page borders, portions and split key ranges."""
    from areal_vllm_amd.ops.attention import alloc_kv_cache

    D = V = 128
    n, device, dtype = 200, "cuda", torch.bfloat16
    pages = [3, 1, 4, 9, 2, 7, 5]
    w_eff = min(window, n)

    def run(h, w, m, portions, nsplit):
        kc, vc = alloc_kv_cache(max(pages) + 2, G, D, dtype, device)
        kc.fill_(50.0)
        vc.fill_(-50.0)
        shape = wattn.ScoreShape(scale=m["scale"], window=window)
        bt = torch.tensor([pages], dtype=torch.int32, device=device)
        r1, r2 = w["r1"].to(dtype).to(device), w["r2"].to(dtype).to(device)
        hd = h.to(dtype).to(device)
        outs, at = [], 0
        for c in portions:
            c = min(c, n - at)
            if c <= 0:
                break
            rows = hd[at:at + c]
            q = wattn.qkv_vnorm_cache_write(rows, _slots(pages, at, at + c, device), kc, vc, H, 1e-6, v_transposed=True,
                                            copy_q=False)
            assert q.data_ptr() == rows.data_ptr()
            gate = rows[:, (H + G) * D + G * V:]
            inside = (at // 7) % 2 == 0  # the gate inside the attention kernels, or as a launch of its own
            o = wattn.window_attention_standard(q, kc, vc, bt, i32([0, c], device), i32([0, at + c], device),
                                                i32([at + c], device), c, shape, nsplit=nsplit if c == 1 else 1,
                                                log_bias=(r1, r2), gate=gate if inside else None).view(c, H * V)
            outs.append((o if inside else wattn.sigmoid_gate_rows(o, gate)).float().cpu())
            at += c
        return torch.cat(outs)

    probes = []
    for qi in (n - 1, 130, 97, 64, 63):
        probes += [(qi, qi - w_eff + 1), (qi, qi - w_eff), (qi, 1), (qi, qi - 32), (qi, qi - 33)]
    probes = [(a, b) for a, b in probes if 0 <= b <= a]
    for k, (qi, kj) in enumerate(probes):
        h, w, m = _window_case(H, G, D, V, window, 4.0 / math.sqrt(D) * 3, n, [(qi, kj)], 7 + k % 3)
        hs = {key: (seen(val, dtype) if key in ("r1", "r2") else val) for key, val in w.items()}
        want = O.window_attention(seen(h, dtype)[:qi + 1], hs, "", m, 1e-6)
        for portions, nsplit in (([n], 1), ([qi, 1, n], 1), ([qi, 1, n], 3)):
            got = run(h, w, m, portions, nsplit)
            assert rel_err(got[qi:qi + 1], want[qi:qi + 1]) < tol(dtype), (qi, kj, portions, nsplit)
    h, w, m = _window_case(H, G, D, V, window, 1.0 / math.sqrt(D), n, [], 1)
    hs = {key: (seen(val, dtype) if key in ("r1", "r2") else val) for key, val in w.items()}
    want = O.window_attention(seen(h, dtype), hs, "", m, 1e-6)
    for portions in ([n], [1], [2], [3, 17, 1, 1, 64, 31, 2, 33, 48], [150, 1]):
        got = run(h, w, m, portions + [portions[-1]] * n, 2)
        assert rel_err(got, want) < tol(dtype), portions


def _latent_case(H, D, P, V, R, n, seed, base=100.0, scale=None, far=None, sink=None):
    """One sequence whose projections are identity-like: the input's columns are the queries and the latent | rotary
    key. `far` = (query position, key position): that key's latent and rotary part are made to answer that query's
    first head, so that its score stands out among hundreds."""
    g = torch.Generator().manual_seed(seed)
    nq = H * (D + P)
    width = nq + R + P
    h = torch.randn(n, width, generator=g)
    eye = torch.eye(width, dtype=F64)
    w = {"q": eye[:nq], "dkv": eye[nq:], "dkv.norm": 1 + 0.2 * torch.randn(R, generator=g, dtype=F64),
         "uk": torch.randn(H * D, R, generator=g, dtype=F64) / math.sqrt(R),
         "uv": torch.randn(H * V, R, generator=g, dtype=F64) / math.sqrt(R),
         "sink": torch.randn(H, generator=g, dtype=F64) if sink is None else torch.full((H,), float(sink), dtype=F64),
         "o": torch.eye(H * V, dtype=F64)}
    m = {"heads": H, "dim": D, "rot_dim": P, "vdim": V, "kv_rank": R, "rot": {"base": base, "dims": P},
         "scale": scale if scale is not None else 1.0 / math.sqrt(D + P)}
    if far is not None:
        qi, kj = far
        # the latent whose expanded key is close to the query's unrotated part (least squares through W_uk)
        uk0 = w["uk"][:D]
        c = torch.linalg.lstsq(uk0, h[qi, :D].to(F64).unsqueeze(1)).solution[:, 0]
        h[kj, nq:nq + R] = (6.0 * c / c.norm() * math.sqrt(R)).float()
    return h, w, m


def _run_latent(h, w, m, dtype, device, portions, pages, nsplit=1, matrix_cores=True, lead=0):
    H, D, P, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n, nq = h.shape[0], H * (D + P)
    cache = lattn.alloc_latent_cache(max(pages) + 2, R, P, dtype, device)
    cache.fill_(30.0)
    table = lattn.rotary_table(m["rot"]["base"], P, n + 1, device)
    bt = torch.tensor([pages], dtype=torch.int32, device=device)
    cw, sink = w["dkv.norm"].to(dtype).to(device), w["sink"].to(dtype).to(device)
    uk, uv = w["uk"].to(dtype).to(device), w["uv"].to(dtype).to(device)
    wide = torch.zeros(n, lead + h.shape[1], dtype=dtype, device=device)
    wide[:, lead:] = h.to(dtype).to(device)
    outs, at = [], 0
    for c in portions:
        c = min(c, n - at)
        if c <= 0:
            break
        rows = wide[at:at + c, lead:]
        pos = i32(list(range(at, at + c)), device)
        lattn.latent_prep(rows[:, nq:], 0, R, P, None, cw, pos, _slots(pages, at, at + c, device), cache, table, 1e-6,
                          neighbours=True)
        q = rows[:, :nq].view(c, H, D + P)
        q_lat = torch.einsum("thd,hdr->thr", q[:, :, :D].float(), uk.float().view(H, D, R)).to(dtype).contiguous()
        o_lat = lattn.latent_attention(q, q_lat, cache, bt, i32([0, c], device), i32([at + c], device), c, D, P,
                                       m["scale"], 0, table, nsplit=nsplit if c == 1 else 1, matrix_cores=matrix_cores,
                                       neighbours=True, sink=sink)
        o = torch.einsum("thr,hvr->thv", o_lat.float(), uv.float().view(H, V, R))
        outs.append(o.reshape(c, H * V).float().cpu())
        at += c
    return torch.cat(outs)


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("H,D,P,V,R", [(3, 8, 4, 6, 12), (2, 16, 16, 16, 16), (1, 4, 2, 4, 5), (6, 32, 16, 24, 80),
                                       (4, 24, 32, 16, 64), (2, 64, 64, 64, 128), (5, 10, 6, 7, 20)])
def test_latent_attention_sink_neighbour_rotation_far_keys_portions_and_splits(device, dtype, H, D, P, V, R):
    n = 200
    pages = [5, 1, 7, 3, 0, 6, 2]
    loose = 3.0 if dtype == torch.bfloat16 else 1.0  # q~ and the expansions pass through 16 bits in this harness

    def reference(h, w):
        ws = {k: (seen(v, dtype) if k in ("dkv.norm", "sink", "uk", "uv") else v) for k, v in w.items()}
        return O.latent_attention(seen(h, dtype), ws, "", m, 1e-6)

    # a key far back whose score stands out, seen from a prompt's portion and from decoded tokens; page borders
    for k, (qi, kj) in enumerate([(199, 0), (199, 1), (180, 31), (180, 32), (129, 33), (64, 0), (63, 62)]):
        h, w, m = _latent_case(H, D, P, V, R, n, 11 + k, far=(qi, kj), scale=2.0 / math.sqrt(D + P))
        want = reference(h, w)
        for portions, nsplit in (([n], 1), ([qi, 1, n], 1), ([qi, 1, n], 4)):
            got = _run_latent(h, w, m, dtype, device, portions, pages, nsplit)
            assert rel_err(got[qi:qi + 1], want[qi:qi + 1]) < loose * tol(dtype), (qi, kj, portions, nsplit)
    # whole sequences cut in several ways on both kernels for prompt portions; the projection's rows at an offset
    h, w, m = _latent_case(H, D, P, V, R, n, 5, base=1000000.0)
    want = reference(h, w)
    for portions, mc, lead in (([n], True, 0), ([n], False, 8), ([1], True, 0), ([2], True, 8),
                               ([3, 17, 1, 1, 64, 31, 2, 33], True, 3), ([150, 1], True, 0)):
        got = _run_latent(h, w, m, dtype, device, portions + [portions[-1]] * n, pages, 3, mc, lead)
        assert rel_err(got, want) < loose * tol(dtype), (portions, mc)
    # a sink that dominates shrinks every row; one that is left out (or counted per key) shows at once
    h, w, m = _latent_case(H, D, P, V, R, 40, 6, sink=4.0)
    want = reference(h, w)
    got = _run_latent(h, w, m, dtype, device, [17] + [1] * 40, pages)
    assert rel_err(got, want) < loose * tol(dtype)
    none = dict(w, sink=torch.full((H,), -60.0, dtype=F64))
    assert rel_err(reference(h, none), want) > 0.5
    # the first token attends to itself and the sink alone
    assert rel_err(got[:1], want[:1]) < loose * tol(dtype)


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("H,D,V,tau,rank", [(3, 16, 24, 16.0, 4), (1, 8, 8, 1.0, 1), (2, 40, 70, 4.0, 8),
                                            (2, 64, 64, 16.0, 16), (1, 128, 32, 2.0, 3), (1, 130, 16, 8.0, 2)])
def test_gla_portions_rows_and_slots_used_again(device, dtype, H, D, V, tau, rank):
    g = torch.Generator().manual_seed(D)
    n, n_slots = 150, 4
    N = 2 * H * D + 2 * H * V
    lead, tail = (8, 8) if D % 16 == 0 else (3, 2)
    wide = torch.randn(n, lead + N + rank + tail, generator=g).to(dtype)
    wn = (1 + 0.2 * torch.randn(V, generator=g)).to(dtype)
    a2 = (2.0 * torch.randn(H * D, rank, generator=g)).to(dtype)
    a2b = (1.0 + torch.randn(H * D, generator=g)).to(dtype)
    eye = torch.eye(N + rank, dtype=F64)
    a, b, c = H * D, 2 * H * D, 2 * H * D + H * V
    w = {"q": eye[:a], "k": eye[a:b], "v": eye[b:c], "g": eye[c:N], "a1": eye[N:], "a2": a2.to(F64), "a2.b": a2b.to(F64),
         "norm": wn.to(F64), "o": torch.eye(H * V, dtype=F64)}
    m = {"heads": H, "dim": D, "vdim": V, "tau": tau}
    want, S_want = O.gla(wide[:, lead:lead + N + rank].to(F64), w, "", m, 1e-5)
    state = gla_ops.alloc_state(n_slots, H, D, V, device)
    state.fill_(1e3)  # what an earlier request left
    pd = wide.to(device)[:, lead:lead + N + rank]
    a2d, a2bd = a2.to(device), a2b.to(device)

    def logits(rows):
        return (rows[:, N:].double() @ a2d.double().t()).float()  # fp32 logits of 16-bit operands

    def run(portions, slot):
        outs, at = [], 0
        for cnt in portions:
            cnt = min(cnt, n - at)
            if cnt <= 0:
                break
            rows = pd[at:at + cnt]
            o = gla_ops.gla_scan(rows, 0, a, b, logits(rows), a2bd, tau, D ** -0.5, i32([0, cnt], device),
                                 i32([at], device), i32([slot], device), state, max_q=cnt)
            outs.append(gla_ops.gla_out(o, rows[:, c:N], wn.to(device), 1e-5).float().cpu())
            at += cnt
        return torch.cat(outs)

    for k, sizes in enumerate(([n], [1] * n, [2] * n, [3, 1, 17, 2, 1, 64, 16, 40, 6], [100, 1] + [1] * n,
                               [64, 64, 22], [16] * n)):
        got = run(sizes, k % n_slots)
        assert rel_err(got, want) < tol(dtype), sizes[:4]
        assert rel_err(state[k % n_slots].reshape(1, -1).cpu(), S_want.reshape(1, -1)) < 1e-4
    # two sequences side by side at different places, beside a row that owns no slot
    state.fill_(-7.0)
    first = run([20], 0)
    before = state.clone()
    both = torch.cat([pd[20:23], pd[:40], pd[:2]]).contiguous()
    o = gla_ops.gla_scan(both, 0, a, b, logits(both), a2bd, tau, D ** -0.5, i32([0, 3, 43, 45], device),
                         i32([20, 0, 0], device), i32([0, 3, -1], device), state, max_q=40)
    out = gla_ops.gla_out(o, both[:, c:N], wn.to(device), 1e-5).float().cpu()
    assert bool((o[43:] == 0).all())
    assert rel_err(torch.cat([first, out[:3]]), want[:23]) < tol(dtype) and rel_err(out[3:43], want[:40]) < tol(dtype)
    assert torch.equal(state[[1, 2]], before[[1, 2]])


@pytest.mark.parametrize("device", DEVICES)
def test_gla_strong_decays_keep_every_exponent_finite(device):
    """Logits far below zero with tau = 1 forget the state within a token: a chunked evaluation that divides by
    cumulative decays would overflow here."""
    H, D, V, n = 2, 16, 8, 70
    g = torch.Generator().manual_seed(1)
    N = 2 * H * D + 2 * H * V
    rows = torch.randn(n, N, generator=g)
    z = torch.full((n, H * D), -60.0)
    z[:, ::3] = 5.0
    z[40:, 1] = -200.0
    eye = torch.eye(N, dtype=F64)
    a, b, c = H * D, 2 * H * D, 2 * H * D + H * V
    # the oracle forms its logits as a product: one input column of ones times the wanted logits
    w = {"q": eye[:a], "k": eye[a:b], "v": eye[b:c], "g": eye[c:], "a1": torch.zeros(1, N, dtype=F64),
         "a2": torch.zeros(H * D, 1, dtype=F64), "norm": torch.ones(V, dtype=F64), "o": torch.eye(H * V, dtype=F64)}
    want = []
    for t0, t1 in ((0, 40), (40, n)):  # the logits change once: two runs of the oracle, the state carried over
        w["a2.b"] = z[t0].to(F64)
        y, S = O.gla(rows[t0:t1].to(F64), w, "", {"heads": H, "dim": D, "vdim": V, "tau": 1.0}, 1e-5,
                     state=None if t0 == 0 else S)
        want.append(y)
    want = torch.cat(want)
    state = gla_ops.alloc_state(1, H, D, V, device)
    rd = rows.to(device)
    o = gla_ops.gla_scan(rd, 0, a, b, z.to(device), None, 1.0, D ** -0.5, i32([0, n], device), i32([0], device),
                         i32([0], device), state, max_q=n)
    assert bool(torch.isfinite(o).all()) and bool(torch.isfinite(state).all())
    got = gla_ops.gla_out(o, rd[:, c:], torch.ones(V, device=device), 1e-5)
    assert rel_err(got.cpu(), want) < 2e-4
    assert rel_err(state[0].reshape(1, -1).cpu(), S.reshape(1, -1)) < 1e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,k,count,keep", [(16, 4, 2, 1), (12, 4, 4, 2), (8, 2, 8, 3), (6, 6, 1, 1), (9, 2, 3, 3),
                                            (130, 5, 10, 4), (64, 8, 8, 8)])
def test_group_limited_choice_of_experts(device, E, k, count, keep):
    g = torch.Generator().manual_seed(E + k)
    z = 2 * torch.randn(40, E, generator=g)
    size = E // count
    if count > 1 and size > 1:
        # the single best expert sits in a group whose second-best is poor: the pair of another group wins
        z[0] = -3.0 - 0.01 * torch.arange(E)
        z[0, 0] = 6.0
        z[0, size], z[0, size + 1] = 2.0, 1.9
    topv, topi = moe_ops.moe_group_topk(z.to(device), min(k, keep * size), count, keep)
    s = torch.sigmoid(z.to(F64))
    for t in range(z.shape[0]):
        want = O.route(s[t], min(k, keep * size), count, keep)
        assert topi[t].tolist() == want, t
        assert torch.allclose(topv[t].cpu().to(F64), s[t][want], atol=1e-6)
    if count > 1 and size > 1 and keep == 1:
        assert 0 not in topi[0].tolist()


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("W,ff,E,top,count,keep,shared", [(48, 20, 6, 2, 3, 2, 12), (24, 8, 3, 3, 1, 1, 0),
                                                          (64, 64, 4, 1, 2, 1, 64), (50, 9, 8, 3, 4, 2, 5),
                                                          (32, 16, 1, 1, 1, 1, 8)])
def test_group_routed_and_shared_experts(device, dtype, W, ff, E, top, count, keep, shared):
    g = torch.Generator().manual_seed(W + E)
    mod = RoutedSwiGLUExperts(W, ff, E, top, shared, dtype, device, scoring="sigmoid", groups=(count, keep),
                              router_bias=False, own_shared_in=True)
    w = {}
    for name, p in mod.named_parameters():
        p.data.copy_((torch.randn(p.shape, generator=g) * (2.0 if name == "router" else 1.0) / math.sqrt(p.shape[-1])))
    w["router"] = mod.router.data.cpu().to(F64)
    for i in range(E):
        w[f"e{i}.gate"], w[f"e{i}.up"] = mod.gate_up.data[i, :ff].cpu().to(F64), mod.gate_up.data[i, ff:].cpu().to(F64)
        w[f"e{i}.down"] = mod.down.data[i].cpu().to(F64)
    e = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top, "groups": {"count": count, "keep": keep}}}
    if shared:
        e["shared"] = {"ff": shared}
        w["shared.gate"], w["shared.up"] = mod.shared_in.data[:shared].cpu().to(F64), mod.shared_in.data[shared:].cpu().to(F64)
        w["shared.down"] = mod.shared_down.data.cpu().to(F64)
    h = torch.randn(23, W, generator=g)
    hc = h.to(dtype).to(device)
    got = mod(None, hc, hc.float())
    want = O.moe(seen(h, dtype), w, "", e)
    assert rows_agree(got.float().cpu(), want, dtype), rel_err(got.float().cpu(), want)


# ------------------------------------------------------------------------------------ the engine
def ffn(kind, ff=24, experts=6, top=2, count=3, keep=2, shared=12):
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": ff}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if count:
        d["router"]["groups"] = {"count": count, "keep": keep}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def attn(heads=4, kv=2, dim=16, vdim=8, window=37, scale=0.4, mlp=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": window}}}


def latent(heads=3, dim=8, rot=4, vdim=6, rank=12, base=10000.0, scale=0.3, mlp=None):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": scale,
                      "rot": {"base": base, "dims": rot}}}


def gla(heads=3, dim=16, vdim=24, tau=8.0, rank=4, mlp=None):
    return {"type": "gla", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": rank}}


def config(layers, width=48, vocab=101, eps=1e-5, mult=0.4, positions=512):
    return {"architecture": "Zusotar", "layers": layers, "max_positions": positions, "norm": {"eps": eps},
            "residual_mult": mult, "vocab": vocab, "width": width}


MIXED = config([attn(mlp=ffn("dense", 40)), latent(mlp=ffn("moe")), gla(mlp=ffn("moe", shared=0)),
                attn(heads=2, kv=2, window=5), gla(heads=2, dim=8, vdim=8, tau=1.5, rank=1),
                latent(heads=2, dim=4, rot=2, vdim=4, rank=5, mlp=ffn("moe", experts=3, top=3, count=0, shared=7))])


def make_engine(cfg_dict, device, dtype, num_pages=40, max_running=4, context=512, score=True, graphs=True):
    cfg = ModelConfig.from_hf_dict(cfg_dict)
    srv = InferenceServerConfig(model_path="", dtype=dtype, context_length=context, max_running_requests=max_running,
                                num_continuous_decode_steps=1, max_prefill_tokens=context,
                                disable_cuda_graph=not graphs)
    eng = NativeInferenceEngine(srv, model_config=cfg, device=torch.device(device), num_pages=num_pages,
                                score_mode=score)
    eng.initialize(load_weights=False)
    weights = {k: v.detach().cpu().to(F64) for k, v in eng.model.checkpoint_tensors().items()}
    return eng, weights


def replay(eng, steps):
    """steps: list of lists of (request id, tokens, wanted places, ends after this step) -> {id: {position: logits}}."""
    out, fed, live = {}, {}, set()
    for step in steps:
        for rid, toks, want, _ in step:
            if rid not in live:
                eng.open_replay(rid)
                live.add(rid)
                fed[rid] = 0
        logits = eng.replay_step([(rid, toks, want) for rid, toks, want, _ in step])
        at = 0
        for rid, toks, want, end in step:
            for w in want:
                out.setdefault(rid, {})[fed[rid] + w] = logits[at]
                at += 1
            fed[rid] += len(toks)
            if end:
                eng.close_replay(rid)
                live.discard(rid)
        assert at == logits.shape[0]
    return out


def cut(rid, tokens, sizes):
    """One request alone, fed in portions of the given sizes (the last size repeats); every position is wanted."""
    steps, at, i = [], 0, 0
    while at < len(tokens):
        c = min(sizes[min(i, len(sizes) - 1)], len(tokens) - at)
        steps.append([(rid, tokens[at:at + c], list(range(c)), at + c == len(tokens))])
        at += c
        i += 1
    return steps


_WANT = {}


def check_against_oracle(got, tokens, weights, cfg_dict, dtype, rid, key=None):
    if key is None or key not in _WANT:
        want, _ = O.forward(cfg_dict, weights, tokens)
        if key is not None:
            _WANT[key] = want
    else:
        want = _WANT[key]
    rows = torch.from_numpy(np.stack([got[rid][p] for p in range(len(tokens))]))
    assert rows_agree(rows, want, dtype), rel_err(rows, want)


def tokens_of(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("device,dtype", CASES)
def test_whole_prompt_and_every_layer(device, dtype):
    eng, w = make_engine(MIXED, device, dtype)
    try:
        toks = tokens_of(75, MIXED["vocab"], 1)
        eng.runner.layer_trace = []
        got = replay(eng, cut("a", toks, [len(toks)]))
        trace, eng.runner.layer_trace = eng.runner.layer_trace, None
        want, layers = O.forward(MIXED, w, toks)
        assert len(trace) == len(layers) == 6
        for a, b in zip(trace, layers):
            assert rows_agree(a.cpu(), b, dtype)
        rows = torch.from_numpy(np.stack([got["a"][p] for p in range(len(toks))]))
        assert rows_agree(rows, want, dtype)
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_prefill_against_token_by_token_and_portions(device, dtype):
    eng, w = make_engine(MIXED, device, dtype)
    try:
        toks = tokens_of(140, MIXED["vocab"], 2)
        for k, sizes in enumerate(([1], [60, 1], [2], [3, 64, 2, 31, 33, 1, 1, 5], [1, 32, 32, 32, 1], [17, 16])):
            got = replay(eng, cut(f"r{k}", toks, list(sizes)))
            check_against_oracle(got, toks, w, MIXED, dtype, f"r{k}", key=("portions", device, dtype))
        assert eng.sched.num_free_state_slots() == 4 and eng.sched.num_free_pages() == eng.sched.num_total_pages()
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(device, dtype):
    """Seven requests of very different lengths through three slots and a pool that cannot hold them all at once:
    portions of some beside single tokens of others; each must equal the request computed alone."""
    eng, w = make_engine(MIXED, device, dtype, num_pages=15, max_running=3)
    try:
        V = MIXED["vocab"]
        reqs = {f"q{i}": tokens_of(n, V, 10 + i) for i, n in enumerate((1, 70, 23, 130, 2, 97, 40))}
        plan = {"q0": [1], "q1": [5, 1, 1, 33, 2, 1], "q2": [23], "q3": [64, 2, 1, 1, 40, 1], "q4": [1, 1], "q5": [31, 33, 1],
                "q6": [2, 1]}
        waiting, live, at, steps = list(reqs), [], {r: 0 for r in reqs}, []
        nth = {r: 0 for r in reqs}
        while waiting or live:
            while waiting and len(live) < 3:
                need = sum((len(reqs[r]) + 31) // 32 for r in live) + (len(reqs[waiting[0]]) + 31) // 32
                if need > 13:
                    break
                live.append(waiting.pop(0))
            step = []
            for r in list(live):
                sizes = plan[r]
                c = min(sizes[min(nth[r], len(sizes) - 1)], len(reqs[r]) - at[r])
                end = at[r] + c == len(reqs[r])
                step.append((r, reqs[r][at[r]:at[r] + c], list(range(c)), end))
                at[r] += c
                nth[r] += 1
                if end:
                    live.remove(r)
            steps.append(step)
        assert max(len(s) for s in steps) == 3 and any(len(t) == 1 for s in steps if len(s) > 1 for _, t, _, _ in s)
        got = replay(eng, steps)
        for r, toks in reqs.items():
            check_against_oracle(got, toks, w, MIXED, dtype, r)
        assert eng.sched.num_free_state_slots() == 3 and eng.sched.num_free_pages() == eng.sched.num_total_pages()
    finally:
        eng.destroy()


SHAPES = [
    # one head everywhere, key size = value size = rotated size = latent size = width of the expert, as many experts as
    # are chosen, one group, a residual factor and a temperature of 1: values that hide mix-ups
    config([attn(1, 1, 16, 16, 33, mlp=ffn("moe", 16, 2, 2, 1, 1, 16)), latent(1, 16, 16, 16, 16, mlp=ffn("dense", 16)),
            gla(1, 16, 16, 1.0, 16)], width=16, mult=1.0),
    # sizes that are no multiples of 8 or of each other, a window of one token and one beyond the sequence, groups of one
    config([gla(5, 12, 20, 3.0, 3, mlp=ffn("moe", 10, 3, 1, 3, 2, 7)), attn(6, 3, 12, 20, 1, 0.11, mlp=ffn("dense", 30)),
            attn(6, 3, 10, 20, 500, 0.9), latent(3, 20, 6, 60, 7, 500.0, mlp=ffn("moe", 20, 7, 3, 0, 0, 0))],
           width=40, vocab=67, eps=1e-3, mult=0.07),
    config([latent(4, 16, 8, 24, 32)], width=24),  # one layer: the average is over two streams
    config([gla(2, 8, 8, 16.0, 2), gla(4, 32, 16, 2.0, 5, mlp=ffn("moe"))], width=56),  # no paged cache at all
    # nothing a multiple of 4: width, head sizes, expert widths, vocabulary
    config([attn(3, 1, 10, 14, 13, mlp=ffn("moe", 9, 4, 2, 2, 1, 5)), gla(7, 6, 5, 5.0, 3, mlp=ffn("dense", 11)),
            latent(3, 6, 2, 14, 9), attn(3, 1, 6, 14, 3)], width=50, vocab=59),
    # sizes the matrix-core paths take
    config([attn(4, 2, 64, 64, 40, mlp=ffn("moe", 64, 4, 2, 2, 1, 64)), latent(4, 32, 32, 32, 64, mlp=ffn("dense", 128)),
            gla(2, 64, 64, 16.0, 16), attn(8, 2, 128, 32, 70, mlp=ffn("dense", 128)), latent(16, 24, 64, 16, 128),
            gla(1, 128, 128, 4.0, 8), attn(4, 2, 128, 128, 50)], width=64),
]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("which", range(len(SHAPES)))
def test_other_sizes_windows_constants_and_orders(device, dtype, which):
    cfg = SHAPES[which]
    eng, w = make_engine(cfg, device, dtype)
    try:
        toks = tokens_of(90, cfg["vocab"], 20 + which)
        key = ("shapes", which, device, dtype)
        check_against_oracle(replay(eng, cut("w", toks, [len(toks)])), toks, w, cfg, dtype, "w", key=key)
        check_against_oracle(replay(eng, cut("c", toks, [7, 2, 33, 1, 1, 20, 1])), toks, w, cfg, dtype, "c", key=key)
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_orders_and_schedules(device, dtype, seed):
    """Random layer lists (mixer kinds and sizes, windows, constants, with and without feed-forward) fed through random
    schedules of up to three live requests: portions of 1 .. 100 tokens, requests that skip steps."""
    import random

    rng = random.Random(seed)
    for case in range(2):
        width, vocab, layers = rng.choice([32, 48, 72]), rng.choice([37, 101]), []
        for _ in range(rng.randint(1, 4)):
            E = rng.choice([2, 6, 9])
            count = rng.choice([c for c in (1, 2, 3) if E % c == 0])
            mlp = rng.choice([ffn("dense", rng.choice([8, 20, 64])),
                              ffn("moe", rng.choice([8, 20, 64]), E, rng.randint(1, E // count), count,
                                  rng.randint(1, count), rng.choice([0, 8, 24])), None])
            kind = rng.choice(["attention", "latent_attention", "gla"])
            if kind == "attention":
                kv = rng.choice([1, 2, 3])
                layers.append(attn(kv * rng.choice([1, 2, 4]), kv, rng.choice([8, 12, 64, 128]),
                                   rng.choice([8, 20, 32, 64, 128]), rng.choice([1, 2, 31, 32, 33, 100, 400]),
                                   rng.choice([0.1, 0.3]), mlp))
            elif kind == "latent_attention":
                layers.append(latent(rng.choice([1, 2, 5]), rng.choice([8, 12, 32]), rng.choice([2, 8, 32]),
                                     rng.choice([8, 20, 32]), rng.choice([7, 16, 64]), rng.choice([100.0, 1000000.0]),
                                     rng.choice([0.1, 0.3]), mlp))
            else:
                layers.append(gla(rng.choice([1, 2, 3]), rng.choice([8, 24, 64, 128]), rng.choice([8, 40, 64, 72]),
                                  rng.choice([1.0, 4.0, 16.0]), rng.choice([1, 4, 16]), mlp))
        cfg = config(layers, width=width, vocab=vocab, eps=rng.choice([1e-5, 1e-6]), mult=rng.choice([0.2, 1.0]))
        reqs = {f"q{i}": tokens_of(rng.choice([1, 2, 17, 97, 150]), vocab, 7 + 100 * case + i)
                for i in range(rng.randint(1, 3))}
        at, steps = {r: 0 for r in reqs}, []
        while any(at[r] < len(t) for r, t in reqs.items()):
            step = []
            for r, t in reqs.items():
                if at[r] < len(t) and rng.random() > 0.2:
                    c = min(rng.choice([1, 1, 1, 2, 3, 16, 31, 33, 64, 100]), len(t) - at[r])
                    step.append((r, t[at[r]:at[r] + c], list(range(c)), at[r] + c == len(t)))
                    at[r] += c
            if step:
                steps.append(step)
        eng, w = make_engine(cfg, device, dtype, num_pages=24, max_running=3)
        try:
            got = replay(eng, steps)
            for r, t in reqs.items():
                check_against_oracle(got, t, w, cfg, dtype, r)
        finally:
            eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_first_tokens_and_long_decoding(device, dtype):
    cfg = config([attn(window=40, mlp=ffn("dense")), gla(), latent(mlp=ffn("moe")), attn(heads=2, kv=2, window=9)])
    eng, w = make_engine(cfg, device, dtype)
    try:
        for n in (1, 2, 3, 5):
            toks = tokens_of(n, cfg["vocab"], 40 + n)
            check_against_oracle(replay(eng, cut(f"s{n}", toks, [1])), toks, w, cfg, dtype, f"s{n}")
            check_against_oracle(replay(eng, cut(f"w{n}", toks, [n])), toks, w, cfg, dtype, f"w{n}")
        toks = tokens_of(230, cfg["vocab"], 44)  # the windows pass over decoded tokens several times
        check_against_oracle(replay(eng, cut("long", toks, [20, 1])), toks, w, cfg, dtype, "long")
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_engine(device, dtype):
    """The engine's own entry point: prompts of unequal length generated together, prefill plans, then decode
    plans (captured graphs on the GPU), more requests than request slots."""
    cfg = config([attn(window=21, mlp=ffn("dense")), gla(mlp=ffn("moe")), latent(),
                  attn(heads=2, kv=1, dim=16, vdim=16, window=70)], vocab=61)
    eng, w = make_engine(cfg, device, dtype, max_running=3, score=False)
    try:
        prompts = [tokens_of(n, cfg["vocab"], 50 + n) for n in (3, 41, 18, 1, 66)]
        res = eng.generate_blocking(prompts, max_new_tokens=12, greedy=True)
        agree = 0
        for p, r in zip(prompts, res):
            assert r.finish_reason == "length" and len(r.output_tokens) == 12
            want = O.greedy(cfg, w, p, 12 if dtype == "float32" else 1)
            if dtype == "float32":
                assert r.output_tokens == want
            else:  # a near-tie (of two tokens, of two experts) may flip under bf16
                agree += r.output_tokens[0] == want[0]
        assert dtype == "float32" or agree >= 4
        assert eng.sched.num_free_state_slots() == 3
    finally:
        eng.destroy()


@pytest.mark.parametrize("device", DEVICES)
def test_served_from_a_checkpoint_directory(device, tmp_path):
    """The framework's own path from a directory with config.json and model.safetensors: the model class is chosen by
    the configuration, the rank of the decay projection by a tensor's shape, the weights come through the engine's
    loader; several decode steps per plan."""
    import json

    from areal_vllm_amd.models import build_model

    cfg_dict = config([attn(2, 1, 8, 16, 9, mlp=ffn("moe", 12, 4, 2, 2, 1, 6)), gla(2, 8, 8, 4.0, 3, mlp=ffn("dense", 20)),
                       latent(2, 8, 4, 8, 10)], width=32, vocab=53, positions=128)
    m = build_model(ModelConfig.from_hf_dict(cfg_dict), dtype=torch.bfloat16)
    m.flatten()
    m.init_weights(seed=9)
    m.save_checkpoint(str(tmp_path))
    with open(tmp_path / "config.json") as f:
        saved = json.load(f)
    for l in saved["layers"]:  # a checkpoint whose configuration does not name the rank
        l["mixer"].pop("decay_rank", None)
    with open(tmp_path / "config.json", "w") as f:
        json.dump(saved, f)
    w = {k: v.to(F64) for k, v in m.checkpoint_tensors().items()}
    srv = InferenceServerConfig(model_path=str(tmp_path), dtype="float32", context_length=128, max_running_requests=2,
                                num_continuous_decode_steps=2)
    eng = NativeInferenceEngine(srv, device=torch.device(device), num_pages=12)
    eng.initialize()
    try:
        prompts = [tokens_of(n, 53, 70 + n) for n in (5, 33, 17)]
        res = eng.generate_blocking(prompts, max_new_tokens=7, greedy=True)
        for p, r in zip(prompts, res):
            assert r.output_tokens == O.greedy(cfg_dict, w, p, 7)
    finally:
        eng.destroy()


def test_http_server_command_line_serves_a_checkpoint(tmp_path):
    """The server's own command line -> engine -> POST /generate, greedy, against the float64 formulation."""
    import asyncio
    import socket
    import threading

    import requests
    from aiohttp import web

    from areal_vllm_amd.inference.server import InferenceServer, build_engine, parse_server_args
    from areal_vllm_amd.models import build_model

    cfg_dict = config([latent(2, 8, 4, 8, 10, mlp=ffn("moe", 12, 6, 2, 3, 1, 6)), gla(2, 8, 8, 2.0, 2),
                       attn(2, 1, 8, 16, 11, mlp=ffn("dense", 20))], width=24, vocab=41, positions=128)
    m = build_model(ModelConfig.from_hf_dict(cfg_dict), dtype=torch.float32)
    m.flatten()
    m.init_weights(seed=13)
    m.save_checkpoint(str(tmp_path))
    w = {k: v.to(F64) for k, v in m.checkpoint_tensors().items()}
    args, srv_cfg = parse_server_args(["--model-path", str(tmp_path), "--device", "cpu", "--num-pages", "16", "--dtype",
                                       "float32", "--context-length", "128", "--max-running-requests", "2"])
    eng = build_engine(args, srv_cfg)
    with socket.socket() as sk:
        sk.bind(("127.0.0.1", 0))
        port = sk.getsockname()[1]
    loop, started = asyncio.new_event_loop(), threading.Event()

    def run():
        asyncio.set_event_loop(loop)
        runner = web.AppRunner(InferenceServer(eng).app)
        loop.run_until_complete(runner.setup())
        loop.run_until_complete(web.TCPSite(runner, "127.0.0.1", port).start())
        started.set()
        loop.run_forever()

    threading.Thread(target=run, daemon=True).start()
    assert started.wait(30)
    try:
        prompt = tokens_of(19, 41, 3)
        r = requests.post(f"http://127.0.0.1:{port}/generate", json={
            "input_ids": prompt, "sampling_params": {"max_new_tokens": 6, "temperature": 0.0}}, timeout=120).json()
        assert r["output_ids"] == O.greedy(cfg_dict, w, prompt, 6)
    finally:
        loop.call_soon_threadsafe(loop.stop)
        eng.destroy()


def test_config_reader_and_checkpoint_save_then_load(tmp_path):
    cfg = ModelConfig.from_hf_dict(SHAPES[1])
    assert cfg.family == "zusotar" and cfg.n_layers == 4 and cfg.has_recurrent_state and not cfg.tie_word_embeddings
    assert cfg.residual_mult == 0.07 and cfg.rms_norm_eps == 1e-3 and cfg.max_position_embeddings == 512
    assert not ModelConfig.from_hf_dict(SHAPES[2]).has_recurrent_state
    from areal_vllm_amd.models import build_model

    m = build_model(cfg, dtype=torch.float32)
    m.flatten()
    m.init_weights(seed=4)
    assert sum(p.numel() for p in m.parameters()) == cfg.n_params()
    assert [b.dwa.numel() for b in m.layers] == [2, 3, 4, 5]
    m.save_checkpoint(str(tmp_path))
    cfg2 = ModelConfig.from_pretrained(str(tmp_path))
    assert cfg2.layers == cfg.layers and cfg2.residual_mult == cfg.residual_mult
    m2 = build_model(cfg2, dtype=torch.float32)
    m2.flatten()
    m2.load_checkpoint(str(tmp_path))
    for (n1, a), (n2, b) in zip(m.checkpoint_tensors().items(), m2.checkpoint_tensors().items()):
        assert n1 == n2 and torch.equal(a, b)
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(config([dict(attn(), type="conv")]))
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(config([latent(rot=3)]))
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(config([attn(mlp=ffn("moe", experts=6, count=4))]))
    with pytest.raises(ValueError):
        bad = gla()
        del bad["mixer"]["decay_rank"]
        ModelConfig.from_hf_dict(config([bad]))
