"""Serving throughput of a layer-list design beside the closest standard transformer of equal size.

For every size a Kuzanex model (window attention : mLSTM layers 1 : 2, xIELU feed-forward) and a Qwen3-style
transformer (grouped-query attention with q/k norm, gated MLP) of the same width, depth, head layout and - through
the width of its MLP - parameter count are served by the rollout engine on random weights: the same prompts, the same
number of new tokens, prefill plans and captured decode graphs. Reported per model: prompt tokens/s over the prefill
plans and generated tokens/s over the decode plans (the engine's own clocks), and the parameters per token.

The Lufivik design (latent attention with a sliding window, routed clamped-GLU experts, sublayers between two layer
norms) is compared the same way with a Qwen3-MoE-style transformer: the same width, depth, heads, experts and experts
per token, its experts as wide as the parameter budget allows.

The Pobelorn design (parallel blocks; window attention on rotated unit-norm queries and keys that keeps the first
tokens, every third layer lightning attention; routed + shared gated experts, the first layer a squared-ReLU MLP) is
compared with the same kind of twin.

The Zusotar design (sublayers between two RMS norms, a learned average over depth; window attention with a logarithmic
distance penalty, latent attention with a sink and gated linear attention in turn; group-routed + shared gated
experts, the first layer a gated MLP) is compared with the same kind of twin.
"""
import json
import sys
import time
from typing import Any, Dict, List

import torch

SIZES = {
    # name: width, layers, heads, kv heads, head size, feed-forward, window
    "w1024": (1024, 6, 8, 2, 128, 4096, 512),
    "w2048": (2048, 6, 16, 4, 128, 8192, 512),
    "w4096": (4096, 3, 32, 8, 128, 14336, 1024),
}
# Lufivik: width, layers, heads, unrotated / rotary / value size per head, query / key-value latent size, window,
# experts, experts per token, expert width
LUFIVIK_SIZES = {
    "w1024": (1024, 4, 8, 64, 32, 64, 384, 256, 512, 16, 2, 512),
    "w2048": (2048, 4, 16, 128, 64, 128, 768, 512, 1024, 32, 4, 768),
    "w4096": (4096, 2, 32, 128, 64, 128, 1536, 512, 1024, 64, 4, 1024),
}
# Pobelorn: width, layers, heads, kv heads, head size (keys, values), rotated coordinates, window, kept first tokens,
# experts, experts per token, expert width, shared expert width
POBELORN_SIZES = {
    "w1024": (1024, 4, 8, 2, 128, 64, 512, 4, 16, 2, 512, 512),
    "w2048": (2048, 4, 16, 4, 128, 64, 1024, 4, 32, 4, 768, 768),
    "w4096": (4096, 2, 32, 8, 128, 64, 1024, 4, 64, 4, 1024, 1024),
}
# Zusotar: width, layers, heads, kv heads, head size of the window attention (keys, values), window, latent attention's
# unrotated / rotary / value size per head and latent size, gla heads / key size / value size / decay rank, experts,
# experts per token, groups, groups kept, expert width, shared expert width
ZUSOTAR_SIZES = {
    "w1024": (1024, 4, 8, 2, 128, 512, 64, 32, 64, 256, 4, 128, 256, 16, 16, 2, 4, 2, 512, 512),
    "w2048": (2048, 4, 16, 4, 128, 1024, 128, 64, 128, 512, 8, 128, 256, 16, 32, 4, 4, 2, 768, 768),
    "w4096": (4096, 3, 32, 8, 128, 1024, 128, 64, 128, 512, 16, 128, 256, 32, 64, 4, 8, 4, 1024, 1024),
}
VOCAB = 32768


def kuzanex_dict(width, layers, heads, kv, dim, ff, window) -> Dict[str, Any]:
    ls = []
    for i in range(layers):
        mlp = {"kind": "dense", "ff": ff}
        if i % 3 == 0:
            ls.append({"type": "attention", "mlp": mlp,
                       "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                                 "softcap": 30.0, "mask": {"size": window}}})
        else:
            ls.append({"type": "mlstm", "mlp": mlp,
                       "mixer": {"heads": heads // 2, "dim": dim, "vdim": 2 * dim, "gate_cap": 12.0}})
    return {"architecture": "Kuzanex", "layers": ls, "norm": {"eps": 1e-5}, "postln_alpha": 2.0, "vocab": VOCAB,
            "width": width}


def lufivik_dict(width, layers, heads, dim, rot, vdim, q_rank, kv_rank, window, experts, top, ff) -> Dict[str, Any]:
    layer = {"type": "latent_attention",
             "mixer": {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                       "scale": (dim + rot) ** -0.5, "rot": {"base": 10000.0, "dims": rot}, "mask": {"size": window}},
             "mlp": {"kind": "moe", "expert": {"ff": ff, "limit": 7.0}, "router": {"experts": experts, "top": top}}}
    return {"architecture": "Lufivik", "layers": [json.loads(json.dumps(layer)) for _ in range(layers)],
            "norm": {"eps": 1e-5}, "canon": {"taps": 4},
            "embedding": {"bigram": {"buckets": 65521, "mul_prev": 36313, "mul_cur": 27191}}, "vocab": VOCAB, "width": width}


def pobelorn_dict(width, layers, heads, kv, dim, rot, window, keep, experts, top, ff, shared) -> Dict[str, Any]:
    moe = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}, "shared": {"ff": shared}}
    ls = []
    for i in range(layers):
        mlp = {"kind": "dense", "ff": 4 * width} if i == 0 and layers > 2 else json.loads(json.dumps(moe))
        if i % 3 == 1:
            ls.append({"type": "lightning", "mlp": mlp,
                       "mixer": {"heads": heads, "dim": dim, "vdim": dim,
                                 "decay": [1.0 - 2.0 ** (-(3.0 + 6.0 * (h + 1) / heads)) for h in range(heads)]}})
        else:
            ls.append({"type": "attention", "mlp": mlp,
                       "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                                 "v_mix": True, "mask": {"size": window, "keep_first": keep},
                                 "rot": {"base": 10000.0, "dims": rot,
                                         "scaling": {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}}}})
    return {"architecture": "Pobelorn", "embedding": {"scale": float(width) ** 0.5}, "layers": ls, "norm": {"eps": 1e-6},
            "vocab": VOCAB, "width": width}


def zusotar_dict(width, layers, heads, kv, dim, window, ldim, rot, lvdim, rank, gheads, gdim, gvdim, grank, experts, top,
                 groups, keep, ff, shared, positions=4096) -> Dict[str, Any]:
    moe = {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared},
           "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    mixers = [
        ("attention", {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                       "mask": {"size": window}}),
        ("latent_attention", {"heads": heads, "dim": ldim, "rot_dim": rot, "vdim": lvdim, "kv_rank": rank,
                              "scale": (ldim + rot) ** -0.5, "rot": {"base": 10000.0, "dims": rot}}),
        ("gla", {"heads": gheads, "dim": gdim, "vdim": gvdim, "tau": 8.0, "decay_rank": grank}),
    ]
    ls = []
    for i in range(layers):
        kind, mixer = mixers[i % 3]
        mlp = {"kind": "dense", "ff": 4 * width} if i == 0 and layers > 3 else json.loads(json.dumps(moe))
        ls.append({"type": kind, "mixer": json.loads(json.dumps(mixer)), "mlp": mlp})
    return {"architecture": "Zusotar", "layers": ls, "max_positions": positions, "norm": {"eps": 1e-5},
            "residual_mult": 0.5, "vocab": VOCAB, "width": width}


def moe_twin_config(lcfg, width, layers, heads, experts, top):
    """Qwen3-MoE-style transformer (grouped-query attention, head size 128, routed SwiGLU experts) with the experts
    as wide as the parameter budget of the Lufivik model allows."""
    from ..models.config import ModelConfig

    dim, kv = 128, max(1, heads // 4)
    body = lcfg.n_params(with_embedding=False)
    attn = width * (heads + 2 * kv) * dim + width * heads * dim
    inter = max(64, int(round((body / layers - attn - width * experts) / (3 * width * experts) / 64)) * 64)
    return ModelConfig(family="qwen3_moe", vocab_size=VOCAB, hidden_size=width, n_layers=layers, n_q_heads=heads,
                       n_kv_heads=kv, head_dim=dim, intermediate_size=inter, moe_intermediate_size=inter,
                       n_experts=experts, n_experts_per_tok=top, norm_topk_prob=True, tie_word_embeddings=False,
                       qkv_bias=False, qk_norm=True, rope_theta=1e6, max_position_embeddings=8192, rms_norm_eps=1e-6)


def twin_config(kcfg, width, layers, heads, kv, dim):
    """Qwen3-style transformer whose gated MLP is as wide as the parameter budget of the Kuzanex model allows."""
    from ..models.config import ModelConfig

    body = kcfg.n_params(with_embedding=False)
    attn = width * (heads + 2 * kv) * dim + width * heads * dim
    inter = max(64, int(round((body / layers - attn) / (3 * width) / 64)) * 64)
    return ModelConfig(family="qwen3", vocab_size=VOCAB, hidden_size=width, n_layers=layers, n_q_heads=heads,
                       n_kv_heads=kv, head_dim=dim, intermediate_size=inter, tie_word_embeddings=False, qkv_bias=False,
                       qk_norm=True, rope_theta=1e6, max_position_embeddings=8192, rms_norm_eps=1e-6)


def measure(cfg, n_prompts: int, prompt_len: int, new_tokens: int, device) -> Dict[str, float]:
    from ..api.cli_args import InferenceServerConfig
    from ..inference.engine import NativeInferenceEngine
    from ..ops.attention import PAGE_SIZE

    ctx = prompt_len + new_tokens + PAGE_SIZE
    srv = InferenceServerConfig(model_path="", dtype="bfloat16", context_length=ctx, max_running_requests=n_prompts,
                                num_continuous_decode_steps=8, max_prefill_tokens=8192, disable_radix_cache=True)
    pages = n_prompts * ((ctx + PAGE_SIZE - 1) // PAGE_SIZE + 1) + 8
    eng = NativeInferenceEngine(srv, model_config=cfg, device=device, num_pages=pages)
    eng.initialize(load_weights=False)
    g = torch.Generator().manual_seed(7)
    out = {}
    try:
        for phase in ("warmup", "timed"):
            prompts = [torch.randint(3, VOCAB, (prompt_len,), generator=g).tolist() for _ in range(n_prompts)]
            before = dict(eng.stats)
            p0 = eng.sched.total_prompt_tokens()
            t0 = time.perf_counter()
            res = eng.generate_blocking(prompts, max_new_tokens=new_tokens, temperature=1.0)
            wall = time.perf_counter() - t0
            gen = sum(len(r.output_tokens) for r in res)
            pt = eng.stats["prefill_time"] - before["prefill_time"]
            dt = eng.stats["decode_time"] - before["decode_time"]
            out = dict(prefill_tok_s=(eng.sched.total_prompt_tokens() - p0) / max(pt, 1e-9),
                       decode_tok_s=(gen - n_prompts) / max(dt, 1e-9), wall_s=wall,
                       prefill_ms=1e3 * pt, decode_ms=1e3 * dt)
    finally:
        eng.destroy()
    return out


def run_pobelorn(sizes: List[str], n_prompts: int, prompt_len: int, new_tokens: int, dev) -> int:
    from ..models.config import ModelConfig

    for name in sizes:
        width, layers, heads, kv, dim, rot, window, keep, experts, top, ff, shared = POBELORN_SIZES[name]
        pcfg = ModelConfig.from_hf_dict(pobelorn_dict(*POBELORN_SIZES[name]))
        tcfg = moe_twin_config(pcfg, width, layers, heads, experts, top)
        row = {"design": "pobelorn", "size": name, "width": width, "layers": layers, "heads": heads, "kv_heads": kv,
               "head_dim": dim, "rot_dims": rot, "window": window, "keep_first": keep, "experts": experts, "top": top,
               "expert_ff": ff, "shared_ff": shared, "twin_expert_ff": tcfg.moe_intermediate_size, "prompts": n_prompts,
               "prompt_len": prompt_len, "new_tokens": new_tokens, "dtype": "bf16", "data": "synthetic"}
        for label, cfg in (("pobelorn", pcfg), ("qwen3_moe_twin", tcfg)):
            m = measure(cfg, n_prompts, prompt_len, new_tokens, dev)
            row[label] = {"params_no_embedding": cfg.n_params(with_embedding=False), **{k: round(v, 1) for k, v in m.items()}}
        row["prefill_ratio"] = round(row["pobelorn"]["prefill_tok_s"] / row["qwen3_moe_twin"]["prefill_tok_s"], 3)
        row["decode_ratio"] = round(row["pobelorn"]["decode_tok_s"] / row["qwen3_moe_twin"]["decode_tok_s"], 3)
        print(json.dumps(row), flush=True)
    return 0


def run_zusotar(sizes: List[str], n_prompts: int, prompt_len: int, new_tokens: int, dev) -> int:
    from ..models.config import ModelConfig

    for name in sizes:
        z = ZUSOTAR_SIZES[name]
        width, layers, heads, experts, top = z[0], z[1], z[2], z[14], z[15]
        zcfg = ModelConfig.from_hf_dict(zusotar_dict(*z))
        tcfg = moe_twin_config(zcfg, width, layers, heads, experts, top)
        row = {"design": "zusotar", "size": name, "width": width, "layers": layers, "heads": heads, "kv_heads": z[3],
               "head_dim": z[4], "window": z[5], "kv_rank": z[9], "rot_dim": z[7], "gla_heads": z[10], "gla_dim": z[11],
               "gla_vdim": z[12], "experts": experts, "top": top, "groups": z[16], "groups_kept": z[17],
               "expert_ff": z[18], "shared_ff": z[19], "twin_expert_ff": tcfg.moe_intermediate_size,
               "prompts": n_prompts, "prompt_len": prompt_len, "new_tokens": new_tokens, "dtype": "bf16",
               "data": "synthetic"}
        for label, cfg in (("zusotar", zcfg), ("qwen3_moe_twin", tcfg)):
            m = measure(cfg, n_prompts, prompt_len, new_tokens, dev)
            row[label] = {"params_no_embedding": cfg.n_params(with_embedding=False), **{k: round(v, 1) for k, v in m.items()}}
        row["prefill_ratio"] = round(row["zusotar"]["prefill_tok_s"] / row["qwen3_moe_twin"]["prefill_tok_s"], 3)
        row["decode_ratio"] = round(row["zusotar"]["decode_tok_s"] / row["qwen3_moe_twin"]["decode_tok_s"], 3)
        print(json.dumps(row), flush=True)
    return 0


def run_lufivik(sizes: List[str], n_prompts: int, prompt_len: int, new_tokens: int, dev) -> int:
    from ..models.config import ModelConfig

    for name in sizes:
        width, layers, heads, dim, rot, vdim, q_rank, kv_rank, window, experts, top, ff = LUFIVIK_SIZES[name]
        lcfg = ModelConfig.from_hf_dict(lufivik_dict(*LUFIVIK_SIZES[name]))
        tcfg = moe_twin_config(lcfg, width, layers, heads, experts, top)
        row = {"design": "lufivik", "size": name, "width": width, "layers": layers, "heads": heads,
               "kv_rank": kv_rank, "rot_dim": rot, "window": window, "experts": experts, "top": top, "expert_ff": ff,
               "twin_expert_ff": tcfg.moe_intermediate_size, "prompts": n_prompts, "prompt_len": prompt_len,
               "new_tokens": new_tokens, "dtype": "bf16", "data": "synthetic"}
        for label, cfg in (("lufivik", lcfg), ("qwen3_moe_twin", tcfg)):
            m = measure(cfg, n_prompts, prompt_len, new_tokens, dev)
            row[label] = {"params_no_embedding": cfg.n_params(with_embedding=False), **{k: round(v, 1) for k, v in m.items()}}
        row["prefill_ratio"] = round(row["lufivik"]["prefill_tok_s"] / row["qwen3_moe_twin"]["prefill_tok_s"], 3)
        row["decode_ratio"] = round(row["lufivik"]["decode_tok_s"] / row["qwen3_moe_twin"]["decode_tok_s"], 3)
        print(json.dumps(row), flush=True)
    return 0


def run(sizes: List[str], n_prompts: int, prompt_len: int, new_tokens: int, device="cuda", design="kuzanex") -> int:
    from ..models.config import ModelConfig

    dev = torch.device(device, 0) if device == "cuda" else torch.device(device)
    if design == "lufivik":
        return run_lufivik(sizes, n_prompts, prompt_len, new_tokens, dev)
    if design == "pobelorn":
        return run_pobelorn(sizes, n_prompts, prompt_len, new_tokens, dev)
    if design == "zusotar":
        return run_zusotar(sizes, n_prompts, prompt_len, new_tokens, dev)
    for name in sizes:
        width, layers, heads, kv, dim, ff, window = SIZES[name]
        kcfg = ModelConfig.from_hf_dict(kuzanex_dict(width, layers, heads, kv, dim, ff, window))
        tcfg = twin_config(kcfg, width, layers, heads, kv, dim)
        row = {"size": name, "width": width, "layers": layers, "heads": heads, "kv_heads": kv, "head_dim": dim,
               "window": window, "prompts": n_prompts, "prompt_len": prompt_len, "new_tokens": new_tokens,
               "dtype": "bf16", "data": "synthetic"}
        for label, cfg in (("kuzanex", kcfg), ("qwen3_twin", tcfg)):
            m = measure(cfg, n_prompts, prompt_len, new_tokens, dev)
            row[label] = {"params_no_embedding": cfg.n_params(with_embedding=False), **{k: round(v, 1) for k, v in m.items()}}
        row["prefill_ratio"] = round(row["kuzanex"]["prefill_tok_s"] / row["qwen3_twin"]["prefill_tok_s"], 3)
        row["decode_ratio"] = round(row["kuzanex"]["decode_tok_s"] / row["qwen3_twin"]["decode_tok_s"], 3)
        print(json.dumps(row), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(run(sys.argv[1:] or list(SIZES), 32, 1024, 64))
