"""Sevazen: a decoder-only stack whose layers are listed one by one in the configuration.  A layer is a mixer and an
optional feed-forward, each normed on its OUTPUT only: x <- x + LN1(mixer(x)), x <- x + LN2(ff(x)) with layer norms
that carry a weight and a bias; the sub-layers read the fp32 residual itself.  Mixers:

  ``attention``    grouped-query softmax attention with biased projections, a short causal convolution on q, k and v,
                   per-head q / k RMS norms, part-rotated heads (half-split pairs, Llama-3.1 frequency scaling), a
                   sliding window and a sink per head in the softmax denominator;
  ``attention_2``  differential attention: two score maps per head over the same values, o = a1 - lambda a2, normed per
                   head; YaRN frequency scaling; keys visible inside the query's chunk only; a sigmoid output gate.

Feed-forwards: dense ``W_down relu(W_up x)^2`` or a mixture of such experts (router with a bias, the best ``top``
logits, softmax over the chosen ones) plus a shared expert behind a sigmoid gate of one number per token.  A layer with
``weights_of: j`` runs layer j's weights with a cache and state of its own.  The last norm is a layer norm as well and
the logits come from the embedding table.

Both mixers are ``layers/masked_attention.py::MaskedSoftmaxAttention`` with other options; pages, state slots, the
scheduler, chunked prefill, batching and sampling are the common ones.

Configuration (``config.json``): ``architecture: "Sevazen"``, ``vocab``, ``width``, ``norm.eps``, ``layers`` (``type``,
``mixer`` sizes, ``mlp`` or null, optional ``weights_of``).
Checkpoint names: ``embed``, ``final.norm[.b]``, ``l<i>.norm1|norm2[.b]``, ``l<i>.mix.q|k|v[.b|.conv|.norm]``,
``l<i>.mix.o|g|sink|lq1|lk1|lq2|lk2``, ``l<i>.mlp.up|down`` (dense) or ``l<i>.mlp.router[.b]|e<j>.up|down|
shared.up|down|sg``.
"""
from __future__ import annotations

import math
import re
from typing import Iterable, Optional

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..layers.basic import LogitsProcessor, ParallelLMHead, VocabParallelEmbedding
from ..layers.hyper_connections import _fp32_param
from ..layers.linear import ColumnParallelLinear, RowParallelLinear, default_weight_loader, set_weight_attrs
from ..layers.masked_attention import MaskedSoftmaxAttention
from ..layers.moe import FusedMoE

ARCHITECTURE = "SevazenForCausalLM"
MIXERS = ("attention", "attention_2")
DEFAULT_CONTEXT = 131072
ACT = "relu2"                          # relu(z)^2, every feed-forward of the design


def is_sevazen_config(d: dict) -> bool:
    return d.get("architecture") == "Sevazen" or ARCHITECTURE in (d.get("architectures") or [])


def weight_owner(layers: list, i: int) -> int:
    """The layer whose tensors layer i runs (itself, or the end of its ``weights_of`` chain)."""
    seen = set()
    while layers[i].get("weights_of") is not None:
        if i in seen:
            raise ValueError(f"layer {i}: weights_of forms a cycle")
        seen.add(i)
        i = int(layers[i]["weights_of"])
        if not 0 <= i < len(layers):
            raise ValueError(f"weights_of names layer {i}, which does not exist")
    return i


def normalise_config(d: dict, model_dir: Optional[str] = None) -> dict:
    """Give the engine the names it reads (hidden_size, vocab_size, heads ...)."""
    d = dict(d)
    layers = d["layers"]
    for i, l in enumerate(layers):
        if l["type"] not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        if l.get("mlp") is not None and l["mlp"].get("kind", "dense") not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind {l['mlp'].get('kind')!r}")
        weight_owner(layers, i)
    mix = [l["mixer"] for l in layers]
    d.update(
        architectures=[ARCHITECTURE], model_type="sevazen", hidden_size=int(d["width"]), vocab_size=int(d["vocab"]),
        num_hidden_layers=len(layers), num_attention_heads=max(int(m["heads"]) for m in mix),
        num_key_value_heads=max(int(m["kv_heads"]) for m in mix),
        head_dim=max(max(int(m["dim"]) * (2 if l["type"] == "attention_2" else 1), int(m["vdim"]))
                     for l, m in zip(layers, mix)),
        tie_word_embeddings=True)
    d.setdefault("max_position_embeddings", DEFAULT_CONTEXT)
    d.setdefault("torch_dtype", "bfloat16")
    return d


def make_mixer(kind: str, m: dict, width: int, eps: float, users: int, quant_config, prefix: str):
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    sc = rot.get("scaling")
    common = dict(bias=True, rot_dims=int(rot.get("dims", 0) or 0), rot_base=float(rot.get("base", 10000.0)),
                  users=users, quant_config=quant_config, prefix=prefix)
    if kind == "attention":
        scaling = dict(kind="llama3", factor=float(sc["factor"]), low=float(sc["low"]), high=float(sc["high"]),
                       original=int(sc["original"])) if sc else None
        return MaskedSoftmaxAttention(width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                      float(m["scale"]), eps, conv_taps=int(m.get("conv", 0) or 0),
                                      window=int(mask.get("size", 0) or 0), sink=True, rot_scaling=scaling, **common)
    # cosines and sines of the scaled frequencies are stretched by 0.1 ln(factor) + 1
    scaling = dict(kind="yarn", factor=float(sc["factor"]), original=int(sc["original"]), fast=float(sc["fast"]),
                   slow=float(sc["slow"]), magnitude=0.1 * math.log(float(sc["factor"])) + 1.0) if sc else None
    return MaskedSoftmaxAttention(width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                  float(m["scale"]), eps, chunk=int(mask.get("size", 0) or 0), maps=2,
                                  diff=float(m["diff"]), gate=True, rot_scaling=scaling, **common)


class SquaredReluMLP(nn.Module):
    """W_down relu(W_up x)^2, no biases."""

    def __init__(self, width: int, ff: int, quant_config, prefix: str):
        super().__init__()
        self.up_proj = ColumnParallelLinear(width, ff, bias=False, quant_config=quant_config, prefix=f"{prefix}.up_proj")
        self.down_proj = RowParallelLinear(ff, width, bias=False, quant_config=quant_config,
                                           prefix=f"{prefix}.down_proj")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down_proj(ops.activation(self.up_proj(x), ACT))


class SevazenMoE(nn.Module):
    """Experts without a gate half, chosen by the largest router logits (fp32, with a bias) and weighted by the softmax
    over the chosen logits; a shared expert for every token behind sigmoid(w_sg . x)."""

    def __init__(self, width: int, spec: dict, quant_config, prefix: str):
        super().__init__()
        r, ex = spec["router"], spec["expert"]
        E, top = int(r["experts"]), int(r["top"])
        if not 1 <= top <= E:
            raise ValueError(f"{prefix}: top {top} of {E} experts")
        sh = spec.get("shared")
        self.num_experts = E
        # one fp32 product for everything that is a dot product with x in 32 bits: the router's rows and, last, the
        # shared expert's gate
        rows = E + (1 if sh else 0)
        self.route_weight = nn.Parameter(torch.zeros((rows, width), dtype=torch.float32), requires_grad=False)
        self.route_bias = nn.Parameter(torch.zeros((rows,), dtype=torch.float32), requires_grad=False)

        def load_rows(param, t, part=0):
            lo, hi = (0, E) if part == 0 else (E, rows)
            param.data[lo:hi].copy_(t.to(torch.float32).reshape(param.data[lo:hi].shape))
        set_weight_attrs(self.route_weight, {"weight_loader": load_rows})
        set_weight_attrs(self.route_bias, {"weight_loader": load_rows})
        self.experts = FusedMoE(E, top, width, int(ex["ff"]), renormalize=True, quant_config=quant_config,
                                prefix=f"{prefix}.experts", activation=ACT, gated=False)
        self.shared = SquaredReluMLP(width, int(sh["ff"]), quant_config, f"{prefix}.shared") if sh else None

    def forward(self, x: torch.Tensor):
        """Returns (routed experts' sum, shared expert's output or None, its gate's logit fp32 [T, 1] or None); the
        caller's residual pass forms routed + shared * sigmoid(gate)."""
        z = ops.fp32_rows_dot(x, self.route_weight, self.route_bias)           # fp32 logits [T, E (+ 1)]
        out = self.experts(x, z[:, : self.num_experts])
        if self.shared is None:
            return out, None, None
        return out, self.shared(x), z[:, self.num_experts:]


class LayerNormParams(nn.Module):
    """Weight and bias of a layer norm (fp32); applied by ``ops.residual_layer_norm``."""

    def __init__(self, width: int):
        super().__init__()
        self.weight = _fp32_param((width,), 1.0)
        self.bias = _fp32_param((width,), 0.0)


class SevazenBlock(nn.Module):
    """The tensors of one layer; ``users`` layers of the stack run them, each with a cache and state of its own."""

    def __init__(self, spec: dict, width: int, eps: float, users: int, quant_config, prefix: str):
        super().__init__()
        self.kind, self.eps = spec["type"], eps
        self.norm1 = LayerNormParams(width)
        self.mixer = make_mixer(spec["type"], spec["mixer"], width, eps, users, quant_config, f"{prefix}.mixer")
        mlp = spec.get("mlp")
        self.has_mlp = mlp is not None
        self.routed = self.has_mlp and mlp.get("kind", "dense") != "dense"
        if self.has_mlp:
            self.norm2 = LayerNormParams(width)
            if mlp.get("kind", "dense") == "dense":
                self.mlp = SquaredReluMLP(width, int(mlp["ff"]), quant_config, f"{prefix}.mlp")
            else:
                self.mlp = SevazenMoE(width, mlp, quant_config, f"{prefix}.mlp")

    def forward(self, x: torch.Tensor, h: torch.Tensor, positions: torch.Tensor, user: int) -> torch.Tensor:
        """``x``: the fp32 residual, updated in place; ``h``: the same values in the activation type.  Returns the
        next layer's ``h``."""
        y = self.mixer(h, positions, user)
        h = ops.residual_layer_norm(x, y, self.norm1.weight, self.norm1.bias, self.eps, y.dtype)
        if self.has_mlp:
            y, y2, gate = self.mlp(h) if self.routed else (self.mlp(h), None, None)
            h = ops.residual_layer_norm(x, y, self.norm2.weight, self.norm2.bias, self.eps, y.dtype, y2, gate)
        return h


class SevazenForCausalLM(nn.Module):
    supports_pp = False
    supports_lora = False
    # convolution states live in per-row slots beside the paged keys and values
    row_state_slots = True
    # kernels outside the common set that this model launches (ops/build.py builds them on first use)
    native_sources = ("masked_attention.hip", "attention.hip", "attention_prefill.hip", "mamba.hip", "moe.hip",
                      "gemm_tile.hip")

    def __init__(self, vllm_config: VllmConfig, prefix: str = ""):
        super().__init__()
        config = vllm_config.model_config.hf_config
        self.config = config
        quant_config = getattr(vllm_config, "quant_config", None)
        width, self.eps = int(config.width), float(config.norm["eps"])
        specs = list(config.layers)
        owners = [weight_owner(specs, i) for i in range(len(specs))]
        for i, o in enumerate(owners):
            if specs[i]["type"] != specs[o]["type"]:
                raise ValueError(f"layer {i} runs the weights of layer {o}, a mixer of another type")
        # (owner, which of the owner's users) in the order the stack runs
        self.runs: list[tuple[int, int]] = []
        count: dict[int, int] = {}
        for o in owners:
            self.runs.append((o, count.get(o, 0)))
            count[o] = count.get(o, 0) + 1
        self.embed_tokens = VocabParallelEmbedding(int(config.vocab), width)
        self.blocks = nn.ModuleDict({
            str(o): SevazenBlock(specs[o], width, self.eps, count[o], quant_config, f"blocks.{o}")
            for o in sorted(count)})
        self.norm = LayerNormParams(width)
        self.lm_head = ParallelLMHead(int(config.vocab), width)
        self.lm_head.tie_weights(self.embed_tokens)
        self.logits_processor = LogitsProcessor(int(config.vocab))

    def get_input_embeddings(self, input_ids):
        return self.embed_tokens(input_ids)

    def forward(self, input_ids, positions, intermediate_tensors=None, inputs_embeds=None):
        h = inputs_embeds if inputs_embeds is not None else self.embed_tokens(input_ids)
        x = h.float().contiguous() if h.dtype != torch.float32 else h.clone()
        for o, user in self.runs:
            h = self.blocks[str(o)](x, h, positions, user)
        return ops.residual_layer_norm(x, None, self.norm.weight, self.norm.bias, self.eps, h.dtype)

    def compute_logits(self, hidden_states):
        return self.logits_processor(self.lm_head, hidden_states).float()

    # checkpoint name -> (parameter name, shard id)
    _MIX = {"q": ("in_proj.weight", 0), "k": ("in_proj.weight", 1), "v": ("in_proj.weight", 2),
            "q.b": ("in_proj.bias", 0), "k.b": ("in_proj.bias", 1), "v.b": ("in_proj.bias", 2),
            "q.conv": ("conv_weight", 0), "k.conv": ("conv_weight", 1), "v.conv": ("conv_weight", 2),
            "q.norm": ("q_norm", None), "k.norm": ("k_norm", None), "sink": ("sink", None),
            "lq1": ("lq1", None), "lk1": ("lk1", None), "lq2": ("lq2", None), "lk2": ("lk2", None),
            "g": ("in_proj.weight", 3), "o": ("o_proj.weight", None)}
    _FF = {"up": "up_proj.weight", "down": "down_proj.weight"}
    _TOP = {"embed": "embed_tokens.weight", "final.norm": "norm.weight", "final.norm.b": "norm.bias"}
    _EXPERT = {"up": ("w13_weight", "w1"), "down": ("w2_weight", "w2")}

    def _target(self, name: str):
        """Returns (parameter name, shard id, expert id) or None."""
        if name in self._TOP:
            return self._TOP[name], None, None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or m.group(1) not in self.blocks:
            return None
        blk, rest = self.blocks[m.group(1)], m.group(2)
        base = f"blocks.{m.group(1)}."
        nm = re.fullmatch(r"(norm[12])(\.b)?", rest)
        if nm:
            return base + nm.group(1) + (".bias" if nm.group(2) else ".weight"), None, None
        part, _, leaf = rest.partition(".")
        if part == "mix" and leaf in self._MIX:
            t, shard = self._MIX[leaf]
            return f"{base}mixer.{t}", shard, None
        if part == "mlp" and blk.has_mlp:
            if isinstance(blk.mlp, SquaredReluMLP):
                return (f"{base}mlp.{self._FF[leaf]}", None, None) if leaf in self._FF else None
            if leaf == "router":
                return f"{base}mlp.route_weight", 0, None
            if leaf == "router.b":
                return f"{base}mlp.route_bias", 0, None
            sub, _, w = leaf.partition(".")
            if sub == "shared" and blk.mlp.shared is not None:
                if w in self._FF:
                    return f"{base}mlp.shared.{self._FF[w]}", None, None
                if w == "sg":
                    return f"{base}mlp.route_weight", 1, None
            em = re.fullmatch(r"e(\d+)", sub)
            if em and w in self._EXPERT and int(em.group(1)) < blk.mlp.experts.global_num_experts:
                t, shard = self._EXPERT[w]
                return f"{base}mlp.experts.{t}", shard, int(em.group(1))
        return None

    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> set[str]:
        params = dict(self.named_parameters())
        loaded: set[str] = set()
        for name, t in weights:
            tgt = self._target(name)
            if tgt is None or tgt[0] not in params:
                raise ValueError(f"checkpoint tensor {name!r} has no place in this model")
            target, shard, expert = tgt
            p = params[target]
            loader = getattr(p, "weight_loader", default_weight_loader)
            if expert is not None:
                loader(p, t, shard, expert)
            elif shard is None:
                loader(p, t)
            else:
                loader(p, t, shard)
            loaded.add(target)
        return loaded
