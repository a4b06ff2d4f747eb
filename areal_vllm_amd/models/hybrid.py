"""Layer-list decoders: every layer names its own token mixer, the residual stream is fp32 and normalised AFTER
each sum. The Kuzanex design is the first member: sliding-window attention with shaped scores and mLSTM layers in
any order, feed-forward blocks with the xIELU activation, one gain per norm.

Layer:      x <- norm1(alpha x + mixer(x));  x <- norm2(alpha x + ff(x))       (sublayers read x itself)
Norm:       z / sqrt(mean(z^2) + eps) * g, g one number.
Output:     logits = head . norm(x).

The Lufivik design is the second member. Its layers sit between two norms each (layer norm with bias):

Layer:      h = norm1(x); x <- x + s1 * norm1b(mixer(h + conv(h)) * sigmoid(W_r1 h + b_r1));  the same around ff
Mixer:      attention through a shared low-rank latent (the cache holds the latent and one rotated key per token)
ff:         routed experts, gated units with clamped pre-activations, softmax router weights as they are
Embedding:  token plus hashed-bigram row, then a norm;  a span of layers may run several times (own caches per pass)

The Pobelorn design is the third member. Its layers are parallel blocks on the fp32 stream (RMS norm with a weight):

Layer:      h = norm1(x); x <- x + mixer(h) + ff(h)                 (one norm, both sublayers read it)
Mixers:     grouped-query attention whose queries and keys are rotated by position (interleaved pairs, stretched
            frequencies) and then brought to unit RMS, behind a sliding window that keeps the first tokens, the values
            mixed with those of the first such layer;  or linear attention with a fixed decay per head (fp32 state)
ff:         squared-ReLU MLP, or routed gated experts (router with bias, softmax over the chosen logits) plus a
            shared expert
Embedding:  table row times a constant; the logits come from the same table

The Zusotar design is the fourth member. Its sublayers sit between two RMS norms (weights stored around zero):

Layer:      x <- x + m norm1b(mixer(norm1(x)));  x <- x + m norm2b(ff(norm2(x)));  then a learned average over depth:
            what goes on is sum_j a[j] X_j over the stream ahead of the first layer and behind every layer so far
Mixers:     causal attention through a shared latent (queries straight from the input, rotated neighbour pairs, one sink
            logit per head in the softmax denominator);  grouped-query window attention without rotation whose values
            have unit RMS, with a learned logarithmic distance penalty and an element-wise sigmoid gate;  gated linear
            attention (a decay per key channel from a low-rank projection, fp32 state)
ff:         gated MLP, or routed gated experts chosen by sigmoid scores among the best groups of experts, weighted by
            the scores as they are, plus a shared expert
Embedding:  table row plus a learned vector per position

The mechanisms are separate modules with their constants as constructor arguments (``WindowAttentionMixer``,
``MLSTMMixer``, ``XieluMLP``, ``LatentAttentionMixer``, ``RoutedGLUExperts``, ``RotaryWindowAttentionMixer``,
``LightningMixer``, ``SquaredReluMLP``, ``RoutedSwiGLUExperts``, ``LogBiasWindowAttentionMixer``, ``GLAMixer``,
``GatedMLP``); what they compute is documented with
their kernels (``ops/window_attention.py``, ``ops/mlstm.py``, ``ops/post_norm.py``, ``ops/latent_attention.py``,
``ops/sandwich.py``, ``ops/lightning.py``, ``ops/parallel_block.py``, ``ops/gla.py``, ``ops/depth_avg.py``). The modules hold parameters and know how to run ONE step on the tensors of a
batch plan; paged caches, state slots and the loop over layers belong to the model runner
(``inference/model_runner.py::HybridModelRunner``).
"""
import dataclasses
import json
import os
from typing import Any, Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..ops import depth_avg as davg
from ..ops import gla as gla_ops
from ..ops import lightning as lightning_ops
from ..ops import mlstm as mlstm_ops
from ..ops import parallel_block as pblock
from ..ops import latent_attention as lattn
from ..ops import moe as moe_ops
from ..ops import post_norm, sandwich, window_attention as wattn
from ..ops.grouped_gemm import grouped_gemm_rows
from .config import ModelConfig
from .transformer import FlatParams


@dataclasses.dataclass
class HybridConfig(ModelConfig):
    """`layers`: one dict per layer, {"type": "attention" | "mlstm", "mixer": {...sizes and constants...},
    "mlp": {"kind": "dense", "ff": F} | None}, as the checkpoint's config.json lists them."""
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)
    postln_alpha: float = 1.0
    design: str = "Kuzanex"
    # "post_norm": norm after every sum; "sandwich": layer norms before and after a sublayer, gated; "parallel": one
    # norm, mixer and feed-forward read it and are added together; "prepost": RMS norms before and after a sublayer,
    # the normed output times `residual_mult` added to the stream, optionally averaged over depth
    block_style: str = "post_norm"
    residual_mult: float = 1.0  # factor on every normed sublayer output ("prepost" designs)
    depth_average: bool = False  # the stream that leaves a layer is a learned average of all streams so far
    embed_scale: float = 1.0  # factor on the embedding rows ("parallel" designs)
    loop: Optional[Dict[str, int]] = None  # layers start .. stop - 1 run `times` times in a row
    canon_taps: int = 0  # taps of the causal convolution on a mixer's input (0: none)
    bigram: Optional[Dict[str, int]] = None  # hashed-bigram embedding: buckets, mul_prev, mul_cur

    @property
    def has_recurrent_state(self) -> bool:
        return (any(l["type"] in ("mlstm", "lightning", "gla") for l in self.layers) or self.canon_taps > 1
                or self.bigram is not None)

    @property
    def layer_runs(self) -> List[int]:
        """Index of the layer whose weights each layer run uses, in execution order."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, k = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(a)) + list(range(a, b)) * k + list(range(b, n))

    def n_params(self, with_embedding: bool = True) -> int:
        if self.block_style == "sandwich":
            return self._n_params_sandwich(with_embedding)
        if self.block_style == "parallel":
            return self._n_params_parallel(with_embedding)
        if self.block_style == "prepost":
            return self._n_params_prepost(with_embedding)
        W, n = self.hidden_size, 1
        for l in self.layers:
            m = l["mixer"]
            if l["type"] == "attention":
                H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
                n += (W + 1) * ((H + G) * D + G * V + H) + 2 * D + H * H + W * H * V
            else:
                H, D, V = m["heads"], m["dim"], m["vdim"]
                n += W * (2 * H * D + 2 * H * V) + 2 * H * (W + 1) + H * V + W * H * V
            n += 1
            if l.get("mlp"):
                n += 2 * W * l["mlp"]["ff"] + W + l["mlp"]["ff"] + 3
        return n + (2 * self.vocab_size * W if with_embedding else 0)

    def _n_params_sandwich(self, with_embedding: bool) -> int:
        W = self.hidden_size
        n = 4 * W  # embedding norm, final norm
        for l in self.layers:
            m = l["mixer"]
            H, D, P, V, Q, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            n += W * (Q + R + P + H) + Q + R + Q * H * (D + P) + R * H * (D + V) + W * H * V
            n += 5 * W + W * W + W + W * max(0, self.canon_taps)
            if l.get("mlp"):
                e = l["mlp"]
                n += e["router"]["experts"] * (W + 3 * W * e["expert"]["ff"]) + 5 * W + W * W + W
        if with_embedding:
            n += 2 * self.vocab_size * W + ((self.bigram["buckets"] + 1) * W if self.bigram else 0)
        return n

    def _n_params_parallel(self, with_embedding: bool) -> int:
        W = self.hidden_size
        n = W  # final norm
        for l in self.layers:
            m = l["mixer"]
            H, D, V = m["heads"], m["dim"], m["vdim"]
            if l["type"] == "attention":
                G = m["kv_heads"]
                n += W * (H * D + G * D + G * V) + W * H * V + 1
            else:
                n += W * (2 * H * D + 2 * H * V) + H * V + W * H * V
            n += W
            e = l.get("mlp")
            if e and e["kind"] == "dense":
                n += 2 * W * e["ff"]
            elif e:
                n += e["router"]["experts"] * (W + 1 + 3 * W * e["expert"]["ff"])
                if e.get("shared"):
                    n += 3 * W * e["shared"]["ff"]
        return n + (self.vocab_size * W if with_embedding else 0)

    def _n_params_prepost(self, with_embedding: bool) -> int:
        W = self.hidden_size
        n = W  # final norm
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            H, D, V = m["heads"], m["dim"], m["vdim"]
            if l["type"] == "attention":
                G = m["kv_heads"]
                n += W * (H * D + G * D + G * V + H * V) + 2 * H + W * H * V
            elif l["type"] == "latent_attention":
                P, R = m["rot_dim"], m["kv_rank"]
                n += W * (H * (D + P) + R + P) + R + R * H * (D + V) + H + W * H * V
            else:
                r = m["decay_rank"]
                n += W * (2 * H * D + 2 * H * V + r) + r * H * D + H * D + V + W * H * V
            n += 2 * W + (i + 2 if self.depth_average else 0)
            e = l.get("mlp")
            if e:
                n += 2 * W
                if e["kind"] == "dense":
                    n += 3 * W * e["ff"]
                else:
                    n += e["router"]["experts"] * (W + 3 * W * e["expert"]["ff"])
                    if e.get("shared"):
                        n += 3 * W * e["shared"]["ff"]
        if with_embedding:
            n += 2 * self.vocab_size * W + (self.max_position_embeddings * W if self.pos_embed == "learned" else 0)
        return n

    def to_hf_dict(self) -> Dict[str, Any]:
        if self.block_style == "prepost":
            layers = json.loads(json.dumps(self.layers))  # gla entries carry `decay_rank` (a checkpoint's shapes give it too)
            return {"architecture": self.design, "layers": layers, "max_positions": self.max_position_embeddings,
                    "norm": {"eps": self.rms_norm_eps}, "residual_mult": self.residual_mult,
                    "vocab": self.vocab_size, "width": self.hidden_size}
        if self.block_style == "parallel":
            return {"architecture": self.design, "embedding": {"scale": self.embed_scale},
                    "layers": json.loads(json.dumps(self.layers)), "norm": {"eps": self.rms_norm_eps},
                    "vocab": self.vocab_size, "width": self.hidden_size}
        if self.block_style == "sandwich":
            d = {"architecture": self.design, "layers": [dict(l) for l in self.layers],
                 "norm": {"eps": self.rms_norm_eps}, "vocab": self.vocab_size, "width": self.hidden_size}
            if self.canon_taps:
                d["canon"] = {"taps": self.canon_taps}
            if self.bigram:
                d["embedding"] = {"bigram": dict(self.bigram)}
            if self.loop:
                d["loop"] = dict(self.loop)
            return d
        layers = [{k: v for k, v in l.items() if k != "second_norm" or v} for l in self.layers]
        return {"architecture": "Kuzanex", "layers": layers, "norm": {"eps": self.rms_norm_eps},
                "postln_alpha": self.postln_alpha, "vocab": self.vocab_size, "width": self.hidden_size}


def kuzanex_config(d: Dict[str, Any]) -> HybridConfig:
    """config.json of a Kuzanex checkpoint -> HybridConfig. Every size and constant is taken from it."""
    layers = []
    for i, l in enumerate(d["layers"]):
        if l["type"] not in ("attention", "mlstm"):
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        layers.append({"type": l["type"], "mixer": dict(l["mixer"]), "mlp": dict(mlp) if mlp is not None else None,
                       "second_norm": bool(l.get("second_norm", False))})
    att = next((l["mixer"] for l in layers if l["type"] == "attention"), None)
    return HybridConfig(
        family="kuzanex", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), n_layers=len(layers),
        n_q_heads=int(att["heads"]) if att else 1, n_kv_heads=int(att["kv_heads"]) if att else 1,
        head_dim=int(att["dim"]) if att else 1, intermediate_size=max([l["mlp"]["ff"] for l in layers if l["mlp"]] or [0]),
        rms_norm_eps=float(d["norm"]["eps"]), max_position_embeddings=int(d.get("max_positions", 1 << 17)),
        tie_word_embeddings=False, qkv_bias=True, qk_norm=True, pos_embed="none", layers=layers,
        postln_alpha=float(d["postln_alpha"]), eos_token_id=d.get("eos_token_id"), pad_token_id=d.get("pad_token_id"))


def kuzanex_config_from_dir(path: str) -> HybridConfig:
    """config.json plus one look at the checkpoint's tensor names (which layers without a feed-forward block own
    a second norm gain)."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = kuzanex_config(json.load(f))
    names = set()
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".safetensors"):
            from safetensors import safe_open

            with safe_open(os.path.join(path, fn), framework="pt") as f:
                names.update(f.keys())
    for i, l in enumerate(cfg.layers):
        if l["mlp"] is None and f"l{i}.norm2" in names:
            l["second_norm"] = True
    return cfg


def lufivik_config(d: Dict[str, Any]) -> HybridConfig:
    """config.json of a Lufivik checkpoint -> HybridConfig. Every size and constant is taken from it."""
    layers = []
    for i, l in enumerate(d["layers"]):
        if l["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp.get("kind") != "moe":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        m = l["mixer"]
        if int(m["rot"]["dims"]) != int(m["rot_dim"]) or int(m["rot_dim"]) % 2:
            raise ValueError(f"layer {i}: the rotary part has rot_dim (an even number of) dimensions")
        layers.append({"type": l["type"], "mixer": json.loads(json.dumps(m)),
                       "mlp": json.loads(json.dumps(mlp)) if mlp is not None else None})
    n = len(layers)
    loop = d.get("loop")
    if loop is not None:
        loop = {k: int(loop[k]) for k in ("start", "stop", "times")}
        if not (0 <= loop["start"] <= loop["stop"] <= n and loop["times"] >= 1):
            raise ValueError(f"loop {loop} does not fit {n} layers")
    big = (d.get("embedding") or {}).get("bigram")
    m0 = layers[0]["mixer"]
    moe = [l["mlp"] for l in layers if l["mlp"]]
    return HybridConfig(
        family="lufivik", design="Lufivik", block_style="sandwich", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), n_layers=n, n_q_heads=int(m0["heads"]), n_kv_heads=1, head_dim=int(m0["dim"]),
        intermediate_size=max([e["expert"]["ff"] for e in moe] or [0]), rms_norm_eps=float(d["norm"]["eps"]),
        max_position_embeddings=int(d.get("max_positions", 1 << 17)), tie_word_embeddings=False, qkv_bias=False,
        pos_embed="none", norm_type="layer", layers=layers, loop=loop,
        canon_taps=int((d.get("canon") or {}).get("taps", 0)),
        bigram={k: int(big[k]) for k in ("buckets", "mul_prev", "mul_cur")} if big else None,
        eos_token_id=d.get("eos_token_id"), pad_token_id=d.get("pad_token_id"))


def lufivik_config_from_dir(path: str) -> HybridConfig:
    with open(os.path.join(path, "config.json")) as f:
        return lufivik_config(json.load(f))


def pobelorn_config(d: Dict[str, Any]) -> HybridConfig:
    """config.json of a Pobelorn checkpoint -> HybridConfig. Every size and constant is taken from it."""
    layers = []
    for i, l in enumerate(d["layers"]):
        if l["type"] not in ("attention", "lightning"):
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        m = l["mixer"]
        if l["type"] == "attention":
            rot = m.get("rot")
            if rot and (int(rot["dims"]) % 2 or int(rot["dims"]) > int(m["dim"])):
                raise ValueError(f"layer {i}: the rotated part is an even number of at most dim coordinates")
            if int(m["heads"]) % int(m.get("kv_heads", m["heads"])):
                raise ValueError(f"layer {i}: heads is not a multiple of kv_heads")
        elif len(m["decay"]) != int(m["heads"]):
            raise ValueError(f"layer {i}: one decay per head is needed")
        layers.append({"type": l["type"], "mixer": json.loads(json.dumps(m)),
                       "mlp": json.loads(json.dumps(mlp)) if mlp is not None else None})
    att = next((l["mixer"] for l in layers if l["type"] == "attention"), None)
    widths = [(e["ff"] if e["kind"] == "dense" else e["expert"]["ff"]) for e in (l["mlp"] for l in layers) if e]
    return HybridConfig(
        family="pobelorn", design="Pobelorn", block_style="parallel", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), n_layers=len(layers), n_q_heads=int(att["heads"]) if att else 1,
        n_kv_heads=int(att.get("kv_heads", att["heads"])) if att else 1, head_dim=int(att["dim"]) if att else 1,
        intermediate_size=max(widths or [0]), rms_norm_eps=float(d["norm"]["eps"]),
        max_position_embeddings=int(d.get("max_positions", 1 << 17)), tie_word_embeddings=True, qkv_bias=False,
        pos_embed="none", layers=layers, embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
        eos_token_id=d.get("eos_token_id"), pad_token_id=d.get("pad_token_id"))


def pobelorn_config_from_dir(path: str) -> HybridConfig:
    with open(os.path.join(path, "config.json")) as f:
        return pobelorn_config(json.load(f))


def zusotar_config(d: Dict[str, Any], decay_ranks: Optional[Dict[int, int]] = None) -> HybridConfig:
    """config.json of a Zusotar checkpoint -> HybridConfig. Every size and constant is taken from it; the rank of a gla
    layer's decay projection is a tensor's shape (`decay_ranks`: layer index -> rank, or `decay_rank` in the layer's
    mixer entry)."""
    layers = []
    for i, l in enumerate(d["layers"]):
        if l["type"] not in ("attention", "latent_attention", "gla"):
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        m = json.loads(json.dumps(l["mixer"]))
        if l["type"] == "attention":
            if int(m["heads"]) % int(m.get("kv_heads", m["heads"])):
                raise ValueError(f"layer {i}: heads is not a multiple of kv_heads")
        elif l["type"] == "latent_attention":
            if int(m["rot"]["dims"]) != int(m["rot_dim"]) or int(m["rot_dim"]) % 2:
                raise ValueError(f"layer {i}: the rotary part has rot_dim (an even number of) dimensions")
        else:
            if decay_ranks and i in decay_ranks:
                m["decay_rank"] = int(decay_ranks[i])
            if "decay_rank" not in m:
                raise ValueError(f"layer {i}: the rank of the decay projection is not known")
        if mlp is not None and mlp["kind"] == "moe":
            g = mlp["router"].get("groups")
            if g and (int(mlp["router"]["experts"]) % int(g["count"]) or not 1 <= int(g["keep"]) <= int(g["count"])):
                raise ValueError(f"layer {i}: the expert groups do not fit the experts")
        layers.append({"type": l["type"], "mixer": m, "mlp": json.loads(json.dumps(mlp)) if mlp is not None else None})
    att = next((l["mixer"] for l in layers), None)
    widths = [(e["ff"] if e["kind"] == "dense" else e["expert"]["ff"]) for e in (l["mlp"] for l in layers) if e]
    return HybridConfig(
        family="zusotar", design="Zusotar", block_style="prepost", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), n_layers=len(layers), n_q_heads=int(att["heads"]) if att else 1,
        n_kv_heads=int(att.get("kv_heads", 1)) if att else 1, head_dim=int(att["dim"]) if att else 1,
        intermediate_size=max(widths or [0]), rms_norm_eps=float(d["norm"]["eps"]),
        max_position_embeddings=int(d["max_positions"]), tie_word_embeddings=False, qkv_bias=False,
        pos_embed="learned", layers=layers, residual_mult=float(d.get("residual_mult", 1.0)), depth_average=True,
        eos_token_id=d.get("eos_token_id"), pad_token_id=d.get("pad_token_id"))


def zusotar_config_from_dir(path: str) -> HybridConfig:
    """config.json plus one look at the checkpoint's tensor shapes (the rank of every decay projection)."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    ranks: Dict[int, int] = {}
    want = {f"l{i}.mix.a1": i for i, l in enumerate(d["layers"]) if l["type"] == "gla"}
    if want:
        from safetensors import safe_open

        for fn in sorted(os.listdir(path)):
            if fn.endswith(".safetensors"):
                with safe_open(os.path.join(path, fn), framework="pt") as f:
                    for name in f.keys():
                        if name in want:
                            ranks[want[name]] = int(f.get_slice(name).get_shape()[0])
    return zusotar_config(d, ranks)


class StepTensors:
    """What one batch plan hands to the mixers (all on the device): rows of the packed token batch (`cu_q`, longest
    row `max_q`), each row's context length after the step, cache slot of every token, page tables, position of each
    row's first token, state slot of each row, and the decode launch's split count / workspace."""

    def __init__(self, cu_q, ctx_len, max_q, slots, block_tables, first_pos, state_slots, nsplit=1, workspace=None,
                 positions=None):
        self.cu_q, self.ctx_len, self.max_q, self.slots = cu_q, ctx_len, int(max_q), slots
        self.block_tables, self.first_pos, self.state_slots = block_tables, first_pos, state_slots
        self.nsplit, self.workspace = int(nsplit), workspace
        self.positions = positions  # position of every token (int32), for mixers that rotate by position
        self._cu_k = None
        self.v_first = None  # this step's values of the first value-sharing attention layer [T, G Dv] (set by it)


    @property
    def cu_k(self) -> torch.Tensor:
        """Cumulative context lengths int32 [B + 1] (formed once per step)."""
        if self._cu_k is None:
            self._cu_k = F.pad(torch.cumsum(self.ctx_len, 0, dtype=torch.int32), (1, 0))
        return self._cu_k


class WindowAttentionMixer(nn.Module):
    """Grouped-query attention on RMS-normalised queries and keys (no rotation), scores through soft cap, distance
    bias and head mixing, sliding window, optional sink, one sigmoid gate per head ahead of the output projection.
    q | k | v | gate come out of ONE projection (the gate rows carry no bias)."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, softcap: float,
                 window: int, slope_exp: float, sink: bool, head_mixing: bool, eps: float, dtype, device):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.V, self.eps = heads, kv_heads, dim, vdim, eps
        self.shape = wattn.ScoreShape(scale=scale, softcap=softcap, slope_exp=slope_exp, window=window, sink=sink)
        n = (heads + kv_heads) * dim + kv_heads * vdim + heads
        self.proj = nn.Parameter(torch.empty(n, width, dtype=dtype, device=device))
        self.proj_bias = nn.Parameter(torch.zeros(n, dtype=dtype, device=device))
        self.q_norm = nn.Parameter(torch.ones(dim, dtype=dtype, device=device))
        self.k_norm = nn.Parameter(torch.ones(dim, dtype=dtype, device=device))
        self.talk = nn.Parameter(torch.eye(heads, dtype=dtype, device=device)) if head_mixing else None
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))

    def cache_shape(self):
        return self.G, self.D, self.V

    def step(self, xc: torch.Tensor, st: StepTensors, cache) -> torch.Tensor:
        kc, vc = cache
        T = xc.shape[0]
        H, G, D, V = self.H, self.G, self.D, self.V
        proj = F.linear(xc, self.proj, self.proj_bias)
        q = wattn.qk_norm_cache_write(proj, self.q_norm, self.k_norm, st.slots, kc, vc, H, self.eps)
        o = wattn.window_attention(q, kc, vc, st.block_tables, st.cu_q, st.ctx_len, st.max_q, self.shape, self.talk,
                                   nsplit=st.nsplit if st.max_q == 1 else 1, workspace=st.workspace,
                                   gate=proj[:, (H + G) * D + G * V:])
        return F.linear(o.view(T, H * V), self.o)


class MLSTMMixer(nn.Module):
    """Matrix-memory recurrence: q | k | v | output gate from one projection, the two log gates from a small one
    with fp32 accumulation, capped by `gate_cap`; per-head RMS norm, weight and sigmoid gate on the read-out."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, dtype, device):
        super().__init__()
        self.H, self.D, self.V, self.cap, self.eps = heads, dim, vdim, gate_cap, eps
        self.proj = nn.Parameter(torch.empty(2 * heads * dim + 2 * heads * vdim, width, dtype=dtype, device=device))
        self.gates = nn.Parameter(torch.empty(2 * heads, width, dtype=dtype, device=device))
        self.gates_bias = nn.Parameter(torch.zeros(2 * heads, dtype=dtype, device=device))
        self.norm = nn.Parameter(torch.ones(heads * vdim, dtype=dtype, device=device))
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))

    def state_shape(self):
        return self.H, self.D, self.V

    def step(self, xc: torch.Tensor, st: StepTensors, state) -> torch.Tensor:
        H, D, V = self.H, self.D, self.V
        proj = F.linear(xc, self.proj)
        ig, fg = mlstm_ops.mlstm_gates(xc, self.gates, self.gates_bias, H, self.cap)
        hbuf, nq, mt = mlstm_ops.mlstm_scan(proj, 0, H * D, 2 * H * D, ig, fg, st.cu_q, st.first_pos, st.state_slots,
                                            state, max_q=st.max_q)
        y = mlstm_ops.mlstm_out(hbuf, nq, mt, proj[:, 2 * H * D + H * V:], self.norm, self.eps)
        return F.linear(y, self.o)


class XieluMLP(nn.Module):
    def __init__(self, width: int, ff: int, dtype, device):
        super().__init__()
        self.up = nn.Parameter(torch.empty(ff, width, dtype=dtype, device=device))
        self.up_bias = nn.Parameter(torch.zeros(ff, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype, device=device))
        self.down_bias = nn.Parameter(torch.zeros(width, dtype=dtype, device=device))
        self.act = nn.Parameter(torch.zeros(2, dtype=dtype, device=device))

    def forward(self, xc: torch.Tensor) -> torch.Tensor:
        return F.linear(post_norm.xielu(F.linear(xc, self.up, self.up_bias), self.act), self.down, self.down_bias)


class LatentAttentionMixer(nn.Module):
    """Attention through a shared low-rank latent (``ops/latent_attention.py``): query latent | key/value latent |
    rotary key part | one gate logit per head come out of ONE projection; the queries are expanded from their
    normalised latent, their unrotated parts are carried into latent space with the key expansion (so the cache's
    latents are scored directly) and the attended latents are expanded to values afterwards."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int,
                 scale: float, window: int, rot_base: float, eps: float, dtype, device, head_gate: bool = True,
                 sink: bool = False, neighbour_pairs: bool = False):
        """`q_rank` = 0: the queries come straight out of the input projection (no query latent, no norm of it).
        `head_gate`: one sigmoid gate per head from the same projection. `sink`: one learned logit per head in the
        softmax denominator. `neighbour_pairs`: rotation pairs are columns (2i, 2i + 1) instead of (i, i + P/2)."""
        super().__init__()
        self.H, self.D, self.P, self.V, self.Q, self.R = heads, dim, rot_dim, vdim, q_rank, kv_rank
        self.scale, self.window, self.rot_base, self.eps = float(scale), int(window), float(rot_base), float(eps)
        self.head_gate, self.neighbour_pairs = bool(head_gate), bool(neighbour_pairs)
        self.n_q = q_rank if q_rank > 0 else heads * (dim + rot_dim)  # leading columns of the projection
        self.proj = nn.Parameter(torch.empty(self.n_q + kv_rank + rot_dim + (heads if head_gate else 0), width,
                                             dtype=dtype, device=device))
        self.c_norm = nn.Parameter(torch.ones(kv_rank, dtype=dtype, device=device))
        self.sink = nn.Parameter(torch.zeros(heads, dtype=dtype, device=device)) if sink else None
        if q_rank > 0:
            self.q_norm = nn.Parameter(torch.ones(q_rank, dtype=dtype, device=device))
            self.uq = nn.Parameter(torch.empty(heads * (dim + rot_dim), q_rank, dtype=dtype, device=device))
        else:
            self.q_norm = self.uq = None
        self.uk = nn.Parameter(torch.empty(heads * dim, kv_rank, dtype=dtype, device=device))
        self.uv = nn.Parameter(torch.empty(heads * vdim, kv_rank, dtype=dtype, device=device))
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))
        self.table: Optional[torch.Tensor] = None  # cosines | sines per position (`prepare`)

    def cache_shape(self):
        return self.R, self.P

    def prepare(self, n_pos: int, tables: Dict[Any, torch.Tensor]):
        """The rotation table for positions below `n_pos`; mixers with the same base and size share one."""
        key = (self.rot_base, self.P, int(n_pos))
        if key not in tables:
            tables[key] = lattn.rotary_table(self.rot_base, self.P, int(n_pos), self.proj.device)
        self.table = tables[key]

    def decode_splits(self, batch: int, max_context: int) -> int:
        return lattn.decode_splits(batch, self.window, max_context, self.H)

    def step(self, hc: torch.Tensor, st: StepTensors, cache: torch.Tensor) -> torch.Tensor:
        T = hc.shape[0]
        H, D, P, V, Q, R, nq = self.H, self.D, self.P, self.V, self.Q, self.R, self.n_q
        proj = F.linear(hc, self.proj)
        if Q > 0:
            cq = lattn.latent_prep(proj, Q, R, P, self.q_norm, self.c_norm, st.positions, st.slots, cache, self.table,
                                   self.eps, self.neighbour_pairs)
            q = F.linear(cq, self.uq).view(T, H, D + P)
        else:  # the queries are the projection's leading columns, read in place
            lattn.latent_prep(proj[:, nq:], 0, R, P, None, self.c_norm, st.positions, st.slots, cache, self.table,
                              self.eps, self.neighbour_pairs)
            q = proj[:, :nq].view(T, H, D + P)
        nsplit = 1
        if st.max_q == 1 and st.nsplit > 1:  # this mixer's own share of the step's key-range splits
            nsplit = min(st.nsplit, self.decode_splits(T, self.table.shape[0] - 1))
        # q~_h = W_uk[h]^T q^n_h: one batched product over the heads
        q_lat = torch.bmm(q[:, :, :D].transpose(0, 1), self.uk.view(H, D, R)).transpose(0, 1).contiguous()
        o_lat = lattn.latent_attention(q, q_lat, cache, st.block_tables, st.cu_q, st.ctx_len, st.max_q, D, P,
                                       self.scale, self.window, self.table,
                                       gate=proj[:, nq + R + P:] if self.head_gate else None,
                                       nsplit=nsplit, workspace=st.workspace, neighbours=self.neighbour_pairs,
                                       sink=self.sink)
        o = torch.bmm(o_lat.transpose(0, 1), self.uv.view(H, V, R).transpose(1, 2)).transpose(0, 1)
        return F.linear(o.reshape(T, H * V), self.o)


class RoutedGLUExperts(nn.Module):
    """Routed experts without biases: softmax over all router logits (an fp32 product on the fp32 normed input when
    the caller has it), the `top` largest scores are the weights as they are; expert: down(g sigmoid(alpha g) (u + 1)) with g = min(gate h, limit), u = clamp(up h,
    -limit, limit). Tokens are sorted by expert and every expert runs on a contiguous slab (grouped kernels, row
    ranges on the device)."""

    def __init__(self, width: int, ff: int, experts: int, top: int, limit: float, alpha: float, dtype, device):
        super().__init__()
        assert 1 <= top <= experts
        self.E, self.k, self.ff, self.limit, self.alpha = experts, top, ff, float(limit), float(alpha)
        self.router = nn.Parameter(torch.empty(experts, width, dtype=dtype, device=device))
        self.gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.empty(experts, width, ff, dtype=dtype, device=device))

    def forward(self, hc: torch.Tensor, h32: Optional[torch.Tensor]) -> torch.Tensor:
        if hc.dtype == torch.float32:
            z = F.linear(hc, self.router)
        elif h32 is not None:  # the norm's fp32 output: the choice of experts does not see the bf16 rounding of h
            z = F.linear(h32, self.router.float())
        elif hc.is_cuda:  # bf16 operands, fp32 accumulation AND fp32 logits
            z = torch.mm(hc, self.router.t(), out_dtype=torch.float32)
        else:
            z = F.linear(hc.float(), self.router.float())
        topv, topi = moe_ops.moe_topk(z, self.k, False, out_dtype=torch.float32)
        order, inv, src_row, offsets = moe_ops.moe_sort(topi.reshape(-1), self.E, self.k)
        xs = moe_ops._gather_rows(hc, src_row)
        a = moe_ops.clamped_glu(grouped_gemm_rows(xs, self.gate_up, offsets), self.limit, self.alpha)
        return moe_ops.combine_rows_w32(grouped_gemm_rows(a, self.down, offsets), inv, topv)


class RotaryWindowAttentionMixer(nn.Module):
    """Grouped-query attention: queries and keys rotated by position on their first `rot_dims` coordinates (pairs of
    neighbours, optionally stretched frequencies), then divided by their root mean square (no weight); scores times
    `scale`; sliding window that keeps the first `keep_first` tokens; ordinary softmax. `v_mix` = "first": this
    layer's values are what later layers mix in; "mix": v <- (1 - lam) v + lam v_first with the learned number `vmix`;
    None: plain values. q | k | v are the first columns of the projection the block hands in."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, keep_first: int,
                 rot: Optional[Dict[str, Any]], v_mix: Optional[str], eps: float, dtype, device):
        super().__init__()
        assert heads % kv_heads == 0 and v_mix in (None, "first", "mix")
        self.H, self.G, self.D, self.V, self.eps = heads, kv_heads, dim, vdim, float(eps)
        self.shape = wattn.ScoreShape(scale=float(scale), window=int(window), keep_first=int(keep_first))
        self.rot = dict(rot) if rot else None
        self.v_mix = v_mix
        self.vmix = nn.Parameter(torch.zeros(1, dtype=dtype, device=device))  # read by "mix" layers only
        self.table: Optional[torch.Tensor] = None
        self.standard = False  # the cache is in the engine's standard layout (`alloc_cache`)

    def in_rows(self) -> int:
        return (self.H + self.G) * self.D + self.G * self.V

    def out_cols(self) -> int:
        return self.H * self.V

    def cache_shape(self):
        return self.G, self.D, self.V

    def alloc_cache(self, num_pages: int, dtype, device):
        """Paged K / V of this layer: the engine's standard layout (and its flash / paged-decode kernels) for bf16
        heads of 128 on the GPU, otherwise token-major pages of any key and value size."""
        from ..ops.attention import alloc_kv_cache

        self.standard = wattn.standard_layout_ok(self.D, self.V, dtype, device) and self.H // self.G <= 16
        if self.standard:
            return alloc_kv_cache(num_pages, self.G, self.D, dtype, device)
        return wattn.alloc_window_cache(num_pages, self.G, self.D, self.V, dtype, device)

    def decode_splits(self, batch: int, max_context: int) -> int:
        if self.standard:
            from ..ops.attention import decode_num_splits

            w = self.shape.window
            span = max_context if w <= 0 else min(w + wattn.PAGE_SIZE + self.shape.keep_first, max_context)
            return decode_num_splits(batch, self.G, span)
        return wattn.decode_splits(batch, self.shape.window, max_context, self.shape.keep_first)

    def prepare(self, n_pos: int, tables: Dict[Any, torch.Tensor], device):
        """The rotation table for positions below `n_pos`; mixers with the same constants share one."""
        if not self.rot:
            return
        sc = self.rot.get("scaling") or None
        key = ("rot", float(self.rot["base"]), int(self.rot["dims"]), int(n_pos),
               tuple(float(sc[k]) for k in ("factor", "original", "fast", "slow")) if sc else None)
        if key not in tables:
            tables[key] = wattn.rotation_table(float(self.rot["base"]), int(self.rot["dims"]), int(n_pos), device, sc)
        self.table = tables[key]

    def step(self, proj: torch.Tensor, st: StepTensors, cache) -> torch.Tensor:
        """proj [T, >= in_rows()] -> attended values [T, H Dv] (ahead of the output projection)."""
        kc, vc = cache
        H, G, D, V = self.H, self.G, self.D, self.V
        vf = lam = None
        if self.v_mix == "first":
            st.v_first = proj[:, (H + G) * D:(H + G) * D + G * V]
        elif self.v_mix == "mix":
            vf, lam = st.v_first, self.vmix
            assert vf is not None and vf.shape[1] == G * V, "the value-sharing layers need equal key/value head layouts"
        q = wattn.rot_norm_cache_write(proj, st.positions, self.table, st.slots, kc, vc, H, self.eps, vf, lam,
                                       v_transposed=self.standard)
        nsplit = st.nsplit if st.max_q == 1 else 1
        if self.standard:
            o = wattn.window_attention_standard(q, kc, vc, st.block_tables, st.cu_q, st.cu_k, st.ctx_len, st.max_q,
                                                self.shape, nsplit=nsplit, workspace=st.workspace)
        else:
            o = wattn.window_attention(q, kc, vc, st.block_tables, st.cu_q, st.ctx_len, st.max_q, self.shape, None,
                                       nsplit=nsplit, workspace=st.workspace)
        return o.view(proj.shape[0], H * V)


class LightningMixer(nn.Module):
    """Linear attention with one fixed decay per head (``ops/lightning.py``): q | k | v | gate are the first columns
    of the projection the block hands in, q, k and v pass through SiLU; the read-outs of all heads are RMS-normed
    together (weight `norm`) and multiplied by sigmoid(gate)."""

    def __init__(self, heads: int, dim: int, vdim: int, decay, eps: float, dtype, device):
        super().__init__()
        self.H, self.D, self.V, self.eps = heads, dim, vdim, float(eps)
        self.register_buffer("decay", torch.tensor([float(x) for x in decay], dtype=torch.float32, device=device),
                             persistent=False)
        self.norm = nn.Parameter(torch.ones(heads * vdim, dtype=dtype, device=device))

    def in_rows(self) -> int:
        return 2 * self.H * self.D + 2 * self.H * self.V

    def out_cols(self) -> int:
        return self.H * self.V

    def state_shape(self):
        return self.H, self.D, self.V

    def step(self, proj: torch.Tensor, st: StepTensors, state: torch.Tensor) -> torch.Tensor:
        H, D, V = self.H, self.D, self.V
        o = lightning_ops.lightning_scan(proj, 0, H * D, 2 * H * D, self.decay, st.cu_q, st.first_pos, st.state_slots,
                                         state, max_q=st.max_q)
        return lightning_ops.lightning_out(o, proj[:, 2 * H * D + H * V:2 * H * D + 2 * H * V], self.norm, self.eps)


class SquaredReluMLP(nn.Module):
    """down(max(up h, 0)^2). The up rows are part of the block's in-projection."""

    def __init__(self, width: int, ff: int, dtype, device):
        super().__init__()
        self.ff = ff
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype, device=device))

    def in_rows(self) -> int:
        return self.ff

    def forward(self, cols: torch.Tensor, hc: torch.Tensor, h32: Optional[torch.Tensor]) -> torch.Tensor:
        return F.linear(pblock.relu2_rows(cols), self.down)


class RoutedSwiGLUExperts(nn.Module):
    """Routed gated experts, down(silu(gate h) * (up h)), no biases: router logits W_r h + b in fp32 (on the fp32
    normed input when the caller has it), the `top` largest are chosen and weighted by the softmax over the chosen
    logits alone. Tokens are sorted by expert and every expert runs on a contiguous slab (grouped kernels, row ranges
    on the device). A shared expert of the same form (`shared_ff` > 0) runs for every token and is added; its
    gate | up rows are part of the block's in-projection."""

    def __init__(self, width: int, ff: int, experts: int, top: int, shared_ff: int, dtype, device,
                 scoring: str = "softmax_chosen", groups=None, router_bias: bool = True, own_shared_in: bool = False):
        """`scoring` = "softmax_chosen": as above. "sigmoid": the scores are sigmoid(logits), the `top` largest are
        chosen and are the weights as they are; with `groups` = (count, keep) the experts form `count` equal groups of
        neighbours, a group scores the sum of its two largest scores and only members of the `keep` best groups can
        be chosen. `own_shared_in`: the shared expert's gate | up rows are a parameter of this module (for blocks
        that have no common in-projection)."""
        super().__init__()
        assert 1 <= top <= experts and scoring in ("softmax_chosen", "sigmoid")
        self.E, self.k, self.ff, self.shared_ff = experts, top, ff, int(shared_ff)
        self.scoring = scoring
        self.groups = (int(groups[0]), int(groups[1])) if groups else (1, 1)
        assert experts % self.groups[0] == 0 and 1 <= self.groups[1] <= self.groups[0]
        self.router = nn.Parameter(torch.empty(experts, width, dtype=dtype, device=device))
        self.router_bias = nn.Parameter(torch.zeros(experts, dtype=dtype, device=device)) if router_bias else None
        self.shared_in = (nn.Parameter(torch.empty(2 * shared_ff, width, dtype=dtype, device=device))
                          if own_shared_in and shared_ff > 0 else None)
        self.gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.empty(experts, width, ff, dtype=dtype, device=device))
        self.shared_down = (nn.Parameter(torch.empty(width, shared_ff, dtype=dtype, device=device))
                            if shared_ff > 0 else None)

    def in_rows(self) -> int:
        return 2 * self.shared_ff

    def forward(self, cols: torch.Tensor, hc: torch.Tensor, h32: Optional[torch.Tensor]) -> torch.Tensor:
        # fp32 products on the norm's fp32 output when there is one, else on its rounding
        z = pblock.router_logits(h32 if h32 is not None else hc.float(), self.router, self.router_bias)
        if self.scoring == "sigmoid":
            topv, topi = moe_ops.moe_group_topk(z, self.k, self.groups[0], self.groups[1])
        else:  # softmax over all logits, the k largest re-normalised: the softmax over the chosen logits
            topv, topi = moe_ops.moe_topk(z, self.k, True, out_dtype=torch.float32)
        order, inv, src_row, offsets = moe_ops.moe_sort(topi.reshape(-1), self.E, self.k)
        xs = moe_ops._gather_rows(hc, src_row)
        a = pblock.glu_rows(grouped_gemm_rows(xs, self.gate_up, offsets))
        y = moe_ops.combine_rows_w32(grouped_gemm_rows(a, self.down, offsets), inv, topv)
        if self.shared_down is not None:
            if self.shared_in is not None:
                cols = F.linear(hc, self.shared_in)
            y = torch.addmm(y, pblock.glu_rows(cols), self.shared_down.t())
        return y


class LogBiasWindowAttentionMixer(nn.Module):
    """Grouped-query attention without rotation (``ops/window_attention.py``): q | k | v | gate come out of ONE
    projection; every value head is divided by its root mean square (no weight) and cached so; the score is
    q . k * scale - r1_h ln(1 + r2_h (i - j)) with two learned numbers per head; sliding window; ordinary softmax; the
    heads' outputs are multiplied element by element with sigmoid(gate) ahead of the output projection."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int,
                 v_norm: bool, eps: float, dtype, device):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.V, self.eps, self.v_norm = heads, kv_heads, dim, vdim, float(eps), bool(v_norm)
        self.shape = wattn.ScoreShape(scale=float(scale), window=int(window))
        self.n_qkv = (heads + kv_heads) * dim + kv_heads * vdim
        self.proj = nn.Parameter(torch.empty(self.n_qkv + heads * vdim, width, dtype=dtype, device=device))
        self.r1 = nn.Parameter(torch.zeros(heads, dtype=dtype, device=device))
        self.r2 = nn.Parameter(torch.zeros(heads, dtype=dtype, device=device))
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))
        self.max_context = 1 << 30
        self.standard = False  # the cache is in the engine's standard layout (`alloc_cache`)

    def cache_shape(self):
        return self.G, self.D, self.V

    def alloc_cache(self, num_pages: int, dtype, device):
        """Paged K / V of this layer: the engine's standard layout (and its flash / paged-decode kernels) for bf16
        heads of 128 on the GPU, otherwise token-major pages of any key and value size."""
        from ..ops.attention import alloc_kv_cache

        self.standard = wattn.standard_layout_ok(self.D, self.V, dtype, device) and self.H // self.G <= 16
        if self.standard:
            return alloc_kv_cache(num_pages, self.G, self.D, dtype, device)
        return wattn.alloc_window_cache(num_pages, self.G, self.D, self.V, dtype, device)

    def prepare(self, n_pos: int, tables: Dict[Any, torch.Tensor], device):
        self.max_context = int(n_pos) - 1

    def decode_splits(self, batch: int, max_context: int) -> int:
        if self.standard:
            from ..ops.attention import decode_num_splits

            w = self.shape.window
            return decode_num_splits(batch, self.G, max_context if w <= 0 else min(w + wattn.PAGE_SIZE, max_context))
        return wattn.decode_splits(batch, self.shape.window, max_context)

    def step(self, hc: torch.Tensor, st: StepTensors, cache) -> torch.Tensor:
        kc, vc = cache
        T = hc.shape[0]
        proj = F.linear(hc, self.proj)
        q = wattn.qkv_vnorm_cache_write(proj, st.slots, kc, vc, self.H, self.eps, self.v_norm,
                                        v_transposed=self.standard, copy_q=not self.standard)
        nsplit = 1
        if st.max_q == 1 and st.nsplit > 1:
            nsplit = min(st.nsplit, self.decode_splits(T, self.max_context))
        if self.standard:
            gate = proj[:, self.n_qkv:]
            fused = gate.stride(0) % 4 == 0 and gate.data_ptr() % 8 == 0  # the kernels read the gate as 8-byte vectors
            o = wattn.window_attention_standard(q, kc, vc, st.block_tables, st.cu_q, st.cu_k, st.ctx_len, st.max_q,
                                                self.shape, nsplit=nsplit, workspace=st.workspace,
                                                log_bias=(self.r1, self.r2),
                                                gate=gate if fused else None).view(T, self.H * self.V)
            return F.linear(o if fused else wattn.sigmoid_gate_rows(o, gate), self.o)
        o = wattn.window_attention(q, kc, vc, st.block_tables, st.cu_q, st.ctx_len, st.max_q, self.shape, None,
                                   nsplit=nsplit, workspace=st.workspace, gate=proj[:, self.n_qkv:],
                                   log_bias=(self.r1, self.r2))
        return F.linear(o.view(T, self.H * self.V), self.o)


class GLAMixer(nn.Module):
    """Gated linear attention (``ops/gla.py``): q | k | v | output gate | the low-rank input of the decay logits come
    out of ONE projection; the decay logits are the low-rank product plus a bias, formed in fp32; per key channel the
    state decays by sigmoid(logit)^(1 / tau); per-head RMS norm (one weight vector shared by the heads) and a SiLU
    gate on the read-out."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, tau: float, decay_rank: int, q_scale: float,
                 eps: float, dtype, device):
        super().__init__()
        self.H, self.D, self.V, self.rank = heads, dim, vdim, int(decay_rank)
        self.tau, self.q_scale, self.eps = float(tau), float(q_scale), float(eps)
        self.n_main = 2 * heads * dim + 2 * heads * vdim
        self.proj = nn.Parameter(torch.empty(self.n_main + self.rank, width, dtype=dtype, device=device))
        self.a2 = nn.Parameter(torch.empty(heads * dim, self.rank, dtype=dtype, device=device))
        self.a2_bias = nn.Parameter(torch.zeros(heads * dim, dtype=dtype, device=device))
        self.norm = nn.Parameter(torch.ones(vdim, dtype=dtype, device=device))
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))

    def state_shape(self):
        return self.H, self.D, self.V

    def step(self, hc: torch.Tensor, st: StepTensors, state: torch.Tensor) -> torch.Tensor:
        H, D, V = self.H, self.D, self.V
        proj = F.linear(hc, self.proj)
        low = proj[:, self.n_main:]
        if low.dtype == torch.float32:
            z = F.linear(low, self.a2)
        elif low.is_cuda:  # 16-bit operands, fp32 accumulation AND fp32 logits
            z = torch.mm(low, self.a2.t(), out_dtype=torch.float32)
        else:
            z = F.linear(low.float(), self.a2.float())
        o = gla_ops.gla_scan(proj, 0, H * D, 2 * H * D, z, self.a2_bias, self.tau, self.q_scale, st.cu_q, st.first_pos,
                             st.state_slots, state, max_q=st.max_q)
        y = gla_ops.gla_out(o, proj[:, 2 * H * D + H * V:self.n_main], self.norm, self.eps)
        return F.linear(y, self.o)


class GatedMLP(nn.Module):
    """down(act(gate h) * (up h)); gate | up are one projection."""

    def __init__(self, width: int, ff: int, act: str, dtype, device):
        super().__init__()
        self.ff, self.act = ff, act
        self.gate_up = nn.Parameter(torch.empty(2 * ff, width, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype, device=device))

    def forward(self, cols, hc: torch.Tensor, h32: Optional[torch.Tensor]) -> torch.Tensor:
        return F.linear(pblock.glu_rows(F.linear(hc, self.gate_up), self.act), self.down)


class PrePostBlock(nn.Module):
    """A layer whose sublayers sit between two RMS norms: x <- x + mult * norm_b(sublayer(norm(x))), for the mixer and
    (when the layer has one) the feed-forward; the norms' weights are stored around zero. With `depth_average` the
    layer owns the weights of the average over all streams so far (`n_streams` of them, its own result last). The
    runner closes every sublayer with one launch that also forms the norm the next sublayer reads."""

    def __init__(self, cfg: HybridConfig, spec: Dict[str, Any], n_streams: int, dtype, device):
        super().__init__()
        W, m, eps = cfg.hidden_size, spec["mixer"], cfg.rms_norm_eps
        self.kind = spec["type"]
        if self.kind == "attention":
            self.mix = LogBiasWindowAttentionMixer(
                W, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m.get("scale", float(m["dim"]) ** -0.5)), int((m.get("mask") or {}).get("size") or 0), True, eps,
                dtype, device)
        elif self.kind == "latent_attention":
            self.mix = LatentAttentionMixer(
                W, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), 0, int(m["kv_rank"]),
                float(m.get("scale", (int(m["dim"]) + int(m["rot_dim"])) ** -0.5)),
                int((m.get("mask") or {}).get("size") or 0), float(m["rot"]["base"]), eps, dtype, device,
                head_gate=False, sink=True, neighbour_pairs=True)
        else:
            self.mix = GLAMixer(W, int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), float(m["tau"]),
                                int(m["decay_rank"]), float(m["dim"]) ** -0.5, eps, dtype, device)

        def vec():
            return nn.Parameter(torch.zeros(W, dtype=dtype, device=device))

        self.norm1, self.norm1b = vec(), vec()
        e = spec.get("mlp")
        self.mlp = None
        if e:
            self.norm2, self.norm2b = vec(), vec()
            if e["kind"] == "dense":
                self.mlp = GatedMLP(W, int(e["ff"]), "silu", dtype, device)
            else:
                g = e["router"].get("groups")
                self.mlp = RoutedSwiGLUExperts(
                    W, int(e["expert"]["ff"]), int(e["router"]["experts"]), int(e["router"]["top"]),
                    int((e.get("shared") or {}).get("ff", 0)), dtype, device, scoring="sigmoid",
                    groups=(int(g["count"]), int(g["keep"])) if g else None, router_bias=False, own_shared_in=True)
        self.needs32 = isinstance(self.mlp, RoutedSwiGLUExperts)  # the router reads the norm's fp32 output
        self.dwa = (nn.Parameter(torch.zeros(n_streams, dtype=dtype, device=device)) if cfg.depth_average else None)

    def state_shape(self):
        return None

    def checkpoint_tensors(self, p: str) -> Dict[str, torch.Tensor]:
        m = self.mix
        out = {p + "norm1": self.norm1.data, p + "norm1b": self.norm1b.data, p + "mix.o": m.o.data}
        if self.dwa is not None:
            out[p + "dwa"] = self.dwa.data
        w = m.proj.data
        if self.kind == "attention":
            a, b = m.H * m.D, (m.H + m.G) * m.D
            out.update({p + "mix.q": w[:a], p + "mix.k": w[a:b], p + "mix.v": w[b:m.n_qkv], p + "mix.g": w[m.n_qkv:],
                        p + "mix.r1": m.r1.data, p + "mix.r2": m.r2.data})
        elif self.kind == "latent_attention":
            out.update({p + "mix.q": w[:m.n_q], p + "mix.dkv": w[m.n_q:], p + "mix.dkv.norm": m.c_norm.data,
                        p + "mix.uk": m.uk.data, p + "mix.uv": m.uv.data, p + "mix.sink": m.sink.data})
        else:
            a, b, c = m.H * m.D, 2 * m.H * m.D, 2 * m.H * m.D + m.H * m.V
            out.update({p + "mix.q": w[:a], p + "mix.k": w[a:b], p + "mix.v": w[b:c], p + "mix.g": w[c:m.n_main],
                        p + "mix.a1": w[m.n_main:], p + "mix.a2": m.a2.data, p + "mix.a2.b": m.a2_bias.data,
                        p + "mix.norm": m.norm.data})
        e, q = self.mlp, p + "mlp."
        if e is not None:
            out[p + "norm2"], out[p + "norm2b"] = self.norm2.data, self.norm2b.data
        if isinstance(e, GatedMLP):
            out[q + "gate"], out[q + "up"], out[q + "down"] = e.gate_up.data[:e.ff], e.gate_up.data[e.ff:], e.down.data
        elif e is not None:
            out[q + "router"] = e.router.data
            for i in range(e.E):
                out[q + f"e{i}.gate"] = e.gate_up.data[i, :e.ff]
                out[q + f"e{i}.up"] = e.gate_up.data[i, e.ff:]
                out[q + f"e{i}.down"] = e.down.data[i]
            if e.shared_down is not None:
                sf = e.shared_ff
                out[q + "shared.gate"], out[q + "shared.up"] = e.shared_in.data[:sf], e.shared_in.data[sf:]
                out[q + "shared.down"] = e.shared_down.data
        return out


class ParallelBlock(nn.Module):
    """A layer whose mixer and feed-forward read the same norm of the stream: ONE projection of the normed input
    yields the mixer's operands and the feed-forward's dense first stage (up rows, or the shared expert's gate | up),
    side by side; the two outputs are returned separately and summed into the stream by the caller's closing kernel."""

    def __init__(self, cfg: HybridConfig, spec: Dict[str, Any], v_mix: Optional[str], dtype, device):
        super().__init__()
        W, m, eps = cfg.hidden_size, spec["mixer"], cfg.rms_norm_eps
        self.kind = spec["type"]
        if self.kind == "attention":
            mask = m.get("mask") or {}
            self.mix = RotaryWindowAttentionMixer(
                int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m.get("scale", float(m["dim"]) ** -0.5)), int(mask.get("size") or 0),
                int(mask.get("keep_first") or 0), m.get("rot"), v_mix, eps, dtype, device)
        else:
            self.mix = LightningMixer(int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), m["decay"], eps,
                                      dtype, device)
        e = spec.get("mlp")
        if not e:
            self.mlp = None
        elif e["kind"] == "dense":
            self.mlp = SquaredReluMLP(W, int(e["ff"]), dtype, device)
        else:
            self.mlp = RoutedSwiGLUExperts(W, int(e["expert"]["ff"]), int(e["router"]["experts"]),
                                           int(e["router"]["top"]), int((e.get("shared") or {}).get("ff", 0)), dtype,
                                           device)
        self.norm1 = nn.Parameter(torch.ones(W, dtype=dtype, device=device))
        self.n_mix = self.mix.in_rows()
        self.w_in = nn.Parameter(torch.empty(self.n_mix + (self.mlp.in_rows() if self.mlp is not None else 0), W,
                                             dtype=dtype, device=device))
        self.o = nn.Parameter(torch.empty(W, self.mix.out_cols(), dtype=dtype, device=device))
        self.needs32 = isinstance(self.mlp, RoutedSwiGLUExperts)  # the router reads the norm's fp32 output

    def step(self, hc: torch.Tensor, h32: Optional[torch.Tensor], st: StepTensors, cache, state):
        """(hc, h32) = norm1 of the stream in the compute dtype and (when asked for) fp32 -> (mixer output, feed-forward
        output or None), both [T, W] in the compute dtype."""
        proj = F.linear(hc, self.w_in)
        y = F.linear(self.mix.step(proj, st, cache if self.kind == "attention" else state), self.o)
        if self.mlp is None:
            return y, None
        return y, self.mlp(proj[:, self.n_mix:], hc, h32)

    def checkpoint_tensors(self, p: str) -> Dict[str, torch.Tensor]:
        m, w = self.mix, self.w_in.data
        out = {p + "norm1": self.norm1.data, p + "mix.o": self.o.data}
        if self.kind == "attention":
            a, b = m.H * m.D, (m.H + m.G) * m.D
            out.update({p + "mix.q": w[:a], p + "mix.k": w[a:b], p + "mix.v": w[b:self.n_mix]})
            out[p + "mix.vmix"] = m.vmix.data.view(())
        else:
            a, b, c = m.H * m.D, 2 * m.H * m.D, 2 * m.H * m.D + m.H * m.V
            out.update({p + "mix.q": w[:a], p + "mix.k": w[a:b], p + "mix.v": w[b:c], p + "mix.g": w[c:self.n_mix],
                        p + "mix.norm": m.norm.data})
        e, q = self.mlp, p + "mlp."
        if isinstance(e, SquaredReluMLP):
            out[q + "up"], out[q + "down"] = w[self.n_mix:], e.down.data
        elif e is not None:
            out[q + "router"], out[q + "router.b"] = e.router.data, e.router_bias.data
            for i in range(e.E):
                out[q + f"e{i}.gate"] = e.gate_up.data[i, :e.ff]
                out[q + f"e{i}.up"] = e.gate_up.data[i, e.ff:]
                out[q + f"e{i}.down"] = e.down.data[i]
            if e.shared_down is not None:
                sf = e.shared_ff
                out[q + "shared.gate"], out[q + "shared.up"] = w[self.n_mix:self.n_mix + sf], w[self.n_mix + sf:]
                out[q + "shared.down"] = e.shared_down.data
        return out


class SandwichBlock(nn.Module):
    """A layer whose sublayers sit between two layer norms, with a sigmoid gate computed from the sublayer's normed
    input, one scale per channel on the result, and a causal convolution on what the mixer reads."""

    def __init__(self, cfg: HybridConfig, spec: Dict[str, Any], dtype, device):
        super().__init__()
        W, m, eps = cfg.hidden_size, spec["mixer"], cfg.rms_norm_eps
        self.kind, self.eps = spec["type"], float(eps)

        def vec(n=W, one=False):
            return nn.Parameter((torch.ones if one else torch.zeros)(n, dtype=dtype, device=device))

        mask = m.get("mask") or {}
        self.mix = LatentAttentionMixer(W, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]),
                                        int(m["q_rank"]), int(m["kv_rank"]),
                                        float(m.get("scale", (int(m["dim"]) + int(m["rot_dim"])) ** -0.5)),
                                        int(mask.get("size") or 0), float(m["rot"]["base"]), eps, dtype, device)
        self.norm1, self.norm1_bias, self.norm1b, self.norm1b_bias = vec(one=True), vec(), vec(one=True), vec()
        self.ls1 = vec(one=True)
        self.rg1 = nn.Parameter(torch.empty(W, W, dtype=dtype, device=device))
        self.rg1_bias = vec()
        self.canon1 = (nn.Parameter(torch.zeros(W, cfg.canon_taps, dtype=dtype, device=device))
                       if cfg.canon_taps > 0 else None)
        e = spec.get("mlp")
        self.mlp = None
        if e:
            self.mlp = RoutedGLUExperts(W, int(e["expert"]["ff"]), int(e["router"]["experts"]), int(e["router"]["top"]),
                                        float(e["expert"]["limit"]), 1.702, dtype, device)
            self.norm2, self.norm2_bias, self.norm2b, self.norm2b_bias = vec(one=True), vec(), vec(one=True), vec()
            self.ls2 = vec(one=True)
            self.rg2 = nn.Parameter(torch.empty(W, W, dtype=dtype, device=device))
            self.rg2_bias = vec()

    def state_shape(self):
        """(taps - 1, width) of the convolution's history, or None."""
        return (self.canon1.shape[1] - 1, self.canon1.shape[0]) if self.canon1 is not None and self.canon1.shape[1] > 1 \
            else None

    def step(self, x32: torch.Tensor, h32: torch.Tensor, hc: torch.Tensor, st: StepTensors, cache, state,
             next_norm) -> Any:
        """x32: the stream; (h32, hc) = norm1(x32) in fp32 and in the compute dtype. Returns the new stream and the
        `next_norm` (weight, bias) of it, again in both forms."""
        dtype = hc.dtype
        gate = F.linear(hc, self.rg1, self.rg1_bias)
        if self.canon1 is not None:
            hc = sandwich.canon_conv(h32, self.canon1, state, st.cu_q, st.first_pos, st.state_slots, dtype)
        y = self.mix.step(hc, st, cache)
        if self.mlp is None:
            return sandwich.gated_norm_add(x32, y, gate, self.norm1b, self.norm1b_bias, self.ls1, self.eps, next_norm)
        x32, h32, hc = sandwich.gated_norm_add(x32, y, gate, self.norm1b, self.norm1b_bias, self.ls1, self.eps,
                                               (self.norm2, self.norm2_bias), want32=True)
        gate = F.linear(hc, self.rg2, self.rg2_bias)
        y = self.mlp(hc, h32)
        return sandwich.gated_norm_add(x32, y, gate, self.norm2b, self.norm2b_bias, self.ls2, self.eps, next_norm)

    def checkpoint_tensors(self, p: str) -> Dict[str, torch.Tensor]:
        m = self.mix
        Q, R, P = m.Q, m.R, m.P
        out = {p + "mix.dq": m.proj.data[:Q], p + "mix.dkv": m.proj.data[Q:Q + R + P],
               p + "mix.g": m.proj.data[Q + R + P:], p + "mix.dq.norm": m.q_norm.data,
               p + "mix.dkv.norm": m.c_norm.data, p + "mix.uq": m.uq.data, p + "mix.uk": m.uk.data,
               p + "mix.uv": m.uv.data, p + "mix.o": m.o.data}
        for k in ("1", "2") if self.mlp is not None else ("1",):
            for nm in ("norm" + k, "norm" + k + "b"):
                out[p + nm] = getattr(self, nm).data
                out[p + nm + ".b"] = getattr(self, nm + "_bias").data
            out[p + "ls" + k] = getattr(self, "ls" + k).data
            out[p + "rg" + k] = getattr(self, "rg" + k).data
            out[p + "rg" + k + ".b"] = getattr(self, "rg" + k + "_bias").data
        if self.canon1 is not None:
            out[p + "canon1"] = self.canon1.data
        if self.mlp is not None:
            e, f = self.mlp, self.mlp.ff
            out[p + "mlp.router"] = e.router.data
            for i in range(e.E):
                out[p + f"mlp.e{i}.gate"] = e.gate_up.data[i, :f]
                out[p + f"mlp.e{i}.up"] = e.gate_up.data[i, f:]
                out[p + f"mlp.e{i}.down"] = e.down.data[i]
        return out


class HybridBlock(nn.Module):
    def __init__(self, cfg: HybridConfig, spec: Dict[str, Any], dtype, device):
        super().__init__()
        W, m, eps = cfg.hidden_size, spec["mixer"], cfg.rms_norm_eps
        self.kind = spec["type"]
        if self.kind == "attention":
            mask = m.get("mask") or {}
            self.mix = WindowAttentionMixer(
                W, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m.get("scale", float(m["dim"]) ** -0.5)), float(m.get("softcap") or 0.0),
                int(mask.get("size") or 0), slope_exp=8.0, sink=True, head_mixing=True, eps=eps, dtype=dtype,
                device=device)
        else:
            self.mix = MLSTMMixer(W, int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])),
                                  float(m.get("gate_cap") or 0.0), eps, dtype, device)
        self.norm1 = nn.Parameter(torch.ones(1, dtype=dtype, device=device))
        self.mlp = XieluMLP(W, int(spec["mlp"]["ff"]), dtype, device) if spec.get("mlp") else None
        # a layer without a feed-forward block ends after norm1, unless its checkpoint carries a second gain
        # (`second_norm`, found by `from_pretrained`): then x <- norm2(alpha x) follows
        second = self.mlp is not None or bool(spec.get("second_norm"))
        self.norm2 = nn.Parameter(torch.ones(1, dtype=dtype, device=device)) if second else None


class HybridDecoder(nn.Module):
    """Parameters of a layer-list decoder in one flat buffer (the rollout engine's weight updates address it), random
    initialisation, checkpoint loading. Inference only; one rank."""

    hybrid = True

    def __init__(self, cfg: HybridConfig, dtype=torch.bfloat16, device="cpu", tp_size: int = 1, tp_rank: int = 0,
                 tp_group=None, **unused):
        super().__init__()
        if tp_size != 1:
            raise NotImplementedError("layer-list decoders are served by one rank")
        self.cfg, self.dtype = cfg, dtype
        self.tp_size, self.tp_rank, self.tp_group, self.ep_group = 1, 0, None, None
        self.has_embed = self.has_head = True
        self.layer_ids = list(range(cfg.n_layers))
        self.vocab_range = (0, cfg.vocab_size)
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device))
        self.sandwich = cfg.block_style == "sandwich"
        self.parallel = cfg.block_style == "parallel"
        self.prepost = cfg.block_style == "prepost"
        self.layer_runs = cfg.layer_runs
        if self.prepost:
            if cfg.loop:
                raise NotImplementedError("depth-averaged layers run once each")
            W = cfg.hidden_size
            self.pos = (nn.Parameter(torch.empty(cfg.max_position_embeddings, W, dtype=dtype, device=device))
                        if cfg.pos_embed == "learned" else None)
            self.layers = nn.ModuleList([PrePostBlock(cfg, spec, i + 2, dtype, device)
                                         for i, spec in enumerate(cfg.layers)])
            self.norm = nn.Parameter(torch.zeros(W, dtype=dtype, device=device))
        elif self.parallel:
            blocks, seen_first = [], False
            for spec in cfg.layers:
                v_mix = None
                if spec["type"] == "attention" and spec["mixer"].get("v_mix"):
                    v_mix, seen_first = ("mix" if seen_first else "first"), True
                blocks.append(ParallelBlock(cfg, spec, v_mix, dtype, device))
                if v_mix == "mix":
                    first = next(b.mix for b in blocks if b.kind == "attention" and b.mix.v_mix == "first")
                    if (first.G, first.V) != (blocks[-1].mix.G, blocks[-1].mix.V):
                        raise ValueError("layers that mix values need the key/value heads and value size of the first")
            self.layers = nn.ModuleList(blocks)
            self.norm = nn.Parameter(torch.ones(cfg.hidden_size, dtype=dtype, device=device))
        elif self.sandwich:
            W = cfg.hidden_size
            self.bigram = (nn.Parameter(torch.empty(cfg.bigram["buckets"] + 1, W, dtype=dtype, device=device))
                           if cfg.bigram else None)
            self.embed_norm = nn.Parameter(torch.ones(W, dtype=dtype, device=device))
            self.embed_norm_bias = nn.Parameter(torch.zeros(W, dtype=dtype, device=device))
            self.layers = nn.ModuleList([SandwichBlock(cfg, spec, dtype, device) for spec in cfg.layers])
            self.norm = nn.Parameter(torch.ones(W, dtype=dtype, device=device))
            self.norm_bias = nn.Parameter(torch.zeros(W, dtype=dtype, device=device))
        else:
            self.layers = nn.ModuleList([HybridBlock(cfg, spec, dtype, device) for spec in cfg.layers])
            self.norm = nn.Parameter(torch.ones(1, dtype=dtype, device=device))
        # designs whose logits come from the embedding table have no second matrix
        self.head = (None if cfg.tie_word_embeddings else
                     nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device)))
        self.flat: Optional[FlatParams] = None
        self.flat_experts = None

    @property
    def head_weight(self) -> torch.Tensor:
        return self.head if self.head is not None else self.embed

    def flatten(self, pad_to: int = 1, expert_pad_to=None) -> FlatParams:
        self.flat = FlatParams(self, self.dtype, next(self.parameters()).device, pad_to)
        return self.flat

    def init_weights(self, seed: int = 0, std: float = 0.02):
        g = torch.Generator(device="cpu").manual_seed(seed)
        W = self.cfg.hidden_size
        for n, p in self.named_parameters():
            leaf = n.rsplit(".", 1)[-1]
            if self.prepost:
                if leaf == "dwa":  # mostly the layer's own result, a little of every earlier stream
                    w = 0.3 * torch.rand(p.shape, generator=g) / p.shape[0]
                    w[-1] = 1.0 - w[:-1].sum()
                    p.data.copy_(w)
                elif leaf == "sink":
                    p.data.copy_(torch.randn(p.shape, generator=g))
                elif leaf == "r1":
                    p.data.copy_(0.2 + 0.6 * torch.rand(p.shape, generator=g))
                elif leaf == "r2":
                    p.data.copy_(0.1 + 0.9 * torch.rand(p.shape, generator=g))
                elif leaf == "a2_bias":
                    p.data.copy_(1.0 + torch.randn(p.shape, generator=g))
                elif n.endswith("mix.norm") or leaf == "c_norm":  # plain weights
                    p.data.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
                elif p.dim() == 1:  # norm weights stored around zero
                    p.data.copy_(0.1 * torch.randn(p.shape, generator=g))
                elif leaf == "pos":
                    p.data.copy_(0.5 * torch.randn(p.shape, generator=g))
                elif leaf == "embed":
                    p.data.copy_(torch.randn(p.shape, generator=g))
                else:
                    p.data.copy_(torch.randn(p.shape, generator=g) / (p.shape[-1] ** 0.5))
            elif self.parallel:
                if leaf == "vmix":
                    p.data.copy_(0.2 + 0.6 * torch.rand(p.shape, generator=g))
                elif leaf == "router_bias":
                    p.data.copy_(0.5 * torch.randn(p.shape, generator=g))
                elif p.dim() == 1:  # norm weights
                    p.data.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
                elif leaf == "embed":  # rows of about unit RMS once the embedding's factor is applied
                    p.data.copy_(torch.randn(p.shape, generator=g) / max(self.cfg.embed_scale, 1e-6))
                else:
                    p.data.copy_(torch.randn(p.shape, generator=g) / (p.shape[-1] ** 0.5))
            elif self.sandwich and leaf != "embed" and (p.dim() == 1 or leaf == "canon1"):
                if leaf.endswith("_bias"):
                    p.data.copy_(0.1 * torch.randn(p.shape, generator=g))
                elif leaf == "canon1":
                    p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
                else:  # norm weights and layer scales
                    p.data.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf == "talk":
                p.data.copy_(torch.eye(p.shape[0]) + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf in ("norm1", "norm2") or n == "norm" or leaf in ("q_norm", "k_norm") or n.endswith("mix.norm"):
                p.data.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf == "act":
                p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
            elif leaf.endswith("bias"):
                p.data.copy_(0.1 * torch.randn(p.shape, generator=g))
            elif leaf == "embed":
                p.data.copy_(torch.randn(p.shape, generator=g))
            else:  # projections: unit-variance outputs for a unit-variance input
                p.data.copy_(torch.randn(p.shape, generator=g) / (p.shape[-1] ** 0.5))
            if leaf == "proj_bias":  # the gate rows of the attention projection have no bias
                p.data[-self._mixer_of(n).H:] = 0

    def _mixer_of(self, name: str):
        return self.layers[int(name.split(".")[1])].mix

    def embed_tokens(self, input_ids, positions=None, scatter: bool = False):
        return ops.embedding(input_ids, self.embed)

    def embed_step(self, input_ids: torch.Tensor, st: StepTensors, prev_tokens: Optional[torch.Tensor]) -> torch.Tensor:
        """Sandwich designs: token ids of a batch plan -> the fp32 stream ahead of the first layer (the embedding's
        bigram part reads and replaces the rows' previous tokens in `prev_tokens`)."""
        big = self.cfg.bigram or {}
        return sandwich.embed_bigram_norm(input_ids, self.embed, self.bigram, int(big.get("mul_prev", 0)),
                                          int(big.get("mul_cur", 0)), self.embed_norm, self.embed_norm_bias,
                                          float(self.cfg.rms_norm_eps), st.cu_q, st.first_pos, st.state_slots,
                                          prev_tokens)

    # ------------------------------------------------------------------------- checkpoint names
    def checkpoint_tensors(self) -> Dict[str, torch.Tensor]:
        """Checkpoint name -> the view of this model's parameters that holds it (fused projections are sliced)."""
        if self.prepost:
            out = {"embed": self.embed.data, "head": self.head.data, "final.norm": self.norm.data}
            if self.pos is not None:
                out["pos"] = self.pos.data
            for i, blk in enumerate(self.layers):
                out.update(blk.checkpoint_tensors(f"l{i}."))
            return out
        if self.parallel:
            out = {"embed": self.embed.data, "final.norm": self.norm.data}
            for i, blk in enumerate(self.layers):
                out.update(blk.checkpoint_tensors(f"l{i}."))
            return out
        if self.sandwich:
            out = {"embed": self.embed.data, "head": self.head.data, "final.norm": self.norm.data,
                   "final.norm.b": self.norm_bias.data, "embed.norm": self.embed_norm.data,
                   "embed.norm.b": self.embed_norm_bias.data}
            if self.bigram is not None:
                out["bigram"] = self.bigram.data
            for i, blk in enumerate(self.layers):
                out.update(blk.checkpoint_tensors(f"l{i}."))
            return out
        out: Dict[str, torch.Tensor] = {"embed": self.embed.data, "head": self.head.data,
                                        "final.norm": self.norm.data.view(())}
        for i, blk in enumerate(self.layers):
            p, m = f"l{i}.", blk.mix
            out[p + "norm1"] = blk.norm1.data.view(())
            if blk.norm2 is not None:
                out[p + "norm2"] = blk.norm2.data.view(())
            if blk.kind == "attention":
                H, G, D, V = m.H, m.G, m.D, m.V
                a, b, c = H * D, (H + G) * D, (H + G) * D + G * V
                for nm, lo, hi in (("q", 0, a), ("k", a, b), ("v", b, c)):
                    out[p + f"mix.{nm}"] = m.proj.data[lo:hi]
                    out[p + f"mix.{nm}.b"] = m.proj_bias.data[lo:hi]
                out[p + "mix.g"] = m.proj.data[c:]
                out[p + "mix.q.norm"], out[p + "mix.k.norm"] = m.q_norm.data, m.k_norm.data
                if m.talk is not None:
                    out[p + "mix.talk"] = m.talk.data
                out[p + "mix.o"] = m.o.data
            else:
                H, D, V = m.H, m.D, m.V
                a, b, c = H * D, 2 * H * D, 2 * H * D + H * V
                for nm, lo, hi in (("q", 0, a), ("k", a, b), ("v", b, c), ("g", c, c + H * V)):
                    out[p + f"mix.{nm}"] = m.proj.data[lo:hi]
                out[p + "mix.i"], out[p + "mix.f"] = m.gates.data[:H], m.gates.data[H:]
                out[p + "mix.i.b"], out[p + "mix.f.b"] = m.gates_bias.data[:H], m.gates_bias.data[H:]
                out[p + "mix.norm"], out[p + "mix.o"] = m.norm.data, m.o.data
            if blk.mlp is not None:
                q = p + "mlp."
                out[q + "up"], out[q + "up.b"] = blk.mlp.up.data, blk.mlp.up_bias.data
                out[q + "down"], out[q + "down.b"] = blk.mlp.down.data, blk.mlp.down_bias.data
                out[q + "act"] = blk.mlp.act.data
        return out

    def checkpoint_optional(self) -> set:
        """Names a checkpoint may leave out: numbers that this model's layers never read."""
        if not self.parallel:
            return set()
        return {f"l{i}.mix.vmix" for i, blk in enumerate(self.layers)
                if blk.kind == "attention" and blk.mix.v_mix != "mix"}

    def assign_named_tensors(self, tensors: Dict[str, torch.Tensor], strict: bool = True):
        views = self.checkpoint_tensors()
        unknown = [n for n in tensors if n not in views]
        if strict and unknown:
            raise KeyError(f"{len(unknown)} tensor(s) map onto no parameter of this model: {sorted(unknown)[:8]}")
        for n, t in tensors.items():
            if n in views:
                v = views[n]
                if tuple(v.shape) != tuple(t.shape):
                    raise ValueError(f"{n}: checkpoint shape {tuple(t.shape)}, model expects {tuple(v.shape)}")
                v.copy_(t.to(v.dtype))

    def load_checkpoint(self, path: str, strict: bool = True):
        from safetensors import safe_open

        files = sorted(f for f in os.listdir(path) if f.endswith(".safetensors"))
        if not files:
            raise FileNotFoundError(f"no safetensors files under {path}")
        seen = set()
        for fn in files:
            with safe_open(os.path.join(path, fn), framework="pt") as f:
                names = list(f.keys())
                self.assign_named_tensors({k: f.get_tensor(k) for k in names}, strict=strict)
                seen.update(names)
        missing = sorted(set(self.checkpoint_tensors()) - seen - self.checkpoint_optional())
        if strict and missing:
            raise KeyError(f"checkpoint lacks {len(missing)} tensor(s): {missing[:8]}")

    def save_checkpoint(self, path: str):
        from safetensors.torch import save_file

        os.makedirs(path, exist_ok=True)
        save_file({k: v.detach().cpu().contiguous().clone() for k, v in self.checkpoint_tensors().items()},
                  os.path.join(path, "model.safetensors"))
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump(self.cfg.to_hf_dict(), f, indent=1)
