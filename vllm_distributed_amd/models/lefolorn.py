"""Lefolorn: a decoder-only stack whose layers are listed one by one in the configuration.  A layer normalises the
fp32 residual once, in groups (the row split into ``norm.groups`` equal parts, each divided by its own root mean
square), and both of its sub-layers read that: h = N(x), x <- x + a1 r1(h) mixer(h) + a2 r2(h) ff(h), with per-channel
layer scales a and per-channel sigmoid gates r(h) = sigmoid(R h + b).  Mixers:

  ``attention``         grouped-query softmax attention with biased projections and per-head q / k RMS norms, no
                        rotation: queries grow with the logarithm of their position, a learned bias per (distance
                        bucket, head) joins the scores, the softmax's denominator holds one more 1, values may be
                        mixed with those of the first such layer, and a sigmoid gate multiplies the heads' outputs;
  ``attention_2``       the same projections and norms with part-rotated heads (neighbouring pairs), scores squashed
                        by cap * tanh(score / cap), a sliding window, ordinary softmax, optional value mixing;
  ``latent_attention``  queries through a normed latent, keys and values up-projected from one normed latent per token
                        plus a rotated key part all heads share, a learned sink per head in the softmax denominator.

Feed-forward: routed gated experts (SiLU) chosen by softmax scores plus a correction, from the best groups of
neighbouring experts only, weighted by the plain scores divided by their sum; the router's last ``identity`` outputs
stand for experts that return their input; a shared expert runs for every token.

The two attention mixers are ``layers/masked_attention.py::MaskedSoftmaxAttention`` with other options, the third is
``layers/latent_attention.py::WindowedLatentAttention``; the experts are ``layers/moe.py::FusedMoE``; pages, the
scheduler, chunked prefill, batching and sampling are the common ones.

Configuration (``config.json``): ``architecture: "Lefolorn"``, ``vocab``, ``width``, ``norm.eps``, ``norm.groups``,
``layers`` (``type``, ``mixer`` sizes and constants, ``mlp`` or null).  The number of distance buckets is the row count
of ``l<i>.mix.rel``.
Checkpoint names: ``embed``, ``head``, ``final.norm``, ``l<i>.norm1|ls1|ls2|rg1[.b]|rg2[.b]``,
``l<i>.mix.q|k|v[.b]|q.norm|k.norm|rel|vmix|g|o`` or ``l<i>.mix.dq[.norm]|uq|dkv[.norm]|uk|uv|sink|o``,
``l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down``.
"""
from __future__ import annotations

import os
import re
from typing import Iterable, Optional

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..layers.basic import LogitsProcessor, ParallelLMHead, VocabParallelEmbedding
from ..layers.hyper_connections import _fp32_param
from ..layers.latent_attention import WindowedLatentAttention
from ..layers.linear import MergedColumnParallelLinear, default_weight_loader
from ..layers.masked_attention import MaskedSoftmaxAttention
from ..layers.moe import FusedMoE
from .llama import LlamaMLP

ARCHITECTURE = "LefolornForCausalLM"
MIXERS = ("attention", "attention_2", "latent_attention")
DEFAULT_CONTEXT = 131072
RENORM_EPS = 1e-20                     # joins the chosen scores' sum before the division


def is_lefolorn_config(d: dict) -> bool:
    return d.get("architecture") == "Lefolorn" or ARCHITECTURE in (d.get("architectures") or [])


def normalise_config(d: dict, model_dir: Optional[str] = None) -> dict:
    """Give the engine the names it reads (hidden_size, vocab_size, heads ...) and complete the mixers' sizes with
    what only a tensor's shape tells (the number of distance buckets)."""
    d = dict(d)
    layers = [dict(l, mixer=dict(l["mixer"])) for l in d["layers"]]
    shapes = {}
    st = os.path.join(model_dir, "model.safetensors") if model_dir else None
    if st and os.path.isfile(st):
        from .loader import read_safetensors_header
        header, _ = read_safetensors_header(st)
        shapes = {k: v["shape"] for k, v in header.items() if k != "__metadata__"}
    for i, l in enumerate(layers):
        kind, m = l["type"], l["mixer"]
        if kind not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        if l.get("mlp") is not None and l["mlp"].get("kind", "moe") != "moe":
            raise ValueError(f"layer {i}: unknown feed-forward kind {l['mlp'].get('kind')!r}")
        if kind == "attention" and m.get("bias_max") is not None:
            name = f"l{i}.mix.rel"
            if name in shapes:
                m["bias_rows"] = int(shapes[name][0])
            elif "bias_rows" not in m:
                raise ValueError(f"layer {i}: the number of distance buckets is neither in the configuration "
                                 f"(bias_rows) nor readable from the shape of {name}")
    heads, kv_heads, dims = [], [], []
    for l in layers:
        m = l["mixer"]
        heads.append(int(m["heads"]))
        if l["type"] == "latent_attention":
            kv_heads.append(1)
            dims.append(int(m["kv_rank"]) + int(m["rot_dim"]))
        else:
            kv_heads.append(int(m["kv_heads"]))
            dims.append(max(int(m["dim"]), int(m["vdim"])))
    d.update(
        layers=layers, architectures=[ARCHITECTURE], model_type="lefolorn", hidden_size=int(d["width"]),
        vocab_size=int(d["vocab"]), num_hidden_layers=len(layers), num_attention_heads=max(heads),
        num_key_value_heads=max(kv_heads), head_dim=max(dims), tie_word_embeddings=False)
    d.setdefault("max_position_embeddings", DEFAULT_CONTEXT)
    d.setdefault("torch_dtype", "bfloat16")
    return d


def make_mixer(kind: str, m: dict, width: int, eps: float, quant_config, prefix: str):
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    if kind == "latent_attention":
        return WindowedLatentAttention(
            width, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
            float(m["scale"]), mask.get("size"), rot.get("base"), int(m["rot_dim"]), eps, 1, quant_config, prefix,
            q_rank=int(m["q_rank"]), sink=True)
    common = dict(bias=True, v_mix=bool(m.get("v_mix")), window=int(mask.get("size", 0) or 0),
                  quant_config=quant_config, prefix=prefix)
    sizes = (width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]), eps)
    if kind == "attention":
        t = m.get("q_temp")
        return MaskedSoftmaxAttention(
            *sizes, gate=True, sink_fixed=0.0, q_temp=(float(t["coef"]), int(t["every"])) if t else None,
            dist_bias=(int(m["bias_rows"]), int(m["bias_max"])) if m.get("bias_max") is not None else None, **common)
    return MaskedSoftmaxAttention(
        *sizes, rot_dims=int(rot.get("dims", 0) or 0), rot_base=float(rot.get("base", 10000.0)),
        rot_pairing="neighbours", softcap=float(m.get("softcap", 0.0) or 0.0), **common)


class LefolornMoE(nn.Module):
    """Routed SiLU-gated experts behind a softmax router with a correction on the choice, group-limited; identity
    outputs; a shared expert.  ``forward`` returns (experts' sum, shared expert's output or None, identity weight per
    token or None): the caller's residual pass adds them up."""

    def __init__(self, width: int, spec: dict, quant_config, prefix: str):
        super().__init__()
        r, ex = spec["router"], spec["expert"]
        E, top, ident = int(r["experts"]), int(r["top"]), int(r.get("identity", 0) or 0)
        groups = r.get("groups") or {}
        count, keep = int(groups.get("count", 1) or 1), int(groups.get("keep", 1) or 1)
        n = E + ident
        if n % count or keep > count or top > (n // count) * keep:
            raise ValueError(f"{prefix}: {n} router outputs, {count} groups (keep {keep}) and top {top} do not fit")
        self.router_weight = _fp32_param((n, width), 0.0)
        self.correction = _fp32_param((n,), 0.0)
        self.experts = FusedMoE(E, top, width, int(ex["ff"]), renormalize=True, use_grouped_topk=True,
                                num_expert_group=count, topk_group=keep, quant_config=quant_config,
                                prefix=f"{prefix}.experts", scoring_func="softmax",
                                e_score_correction_bias=self.correction, activation="silu", group_score="max",
                                num_identity_experts=ident, renorm_eps=RENORM_EPS, add_identity=False)
        self.identity = ident
        sh = spec.get("shared")
        self.shared = LlamaMLP(width, int(sh["ff"]), False, quant_config, f"{prefix}.shared") if sh else None

    def forward(self, x: torch.Tensor):
        logits = ops.fp32_rows_dot(x, self.router_weight)                     # the router runs in fp32
        out = self.experts(x, logits)
        return (out, self.shared(x) if self.shared is not None else None,
                self.experts.identity_weight if self.identity else None)


class LefolornLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, quant_config, prefix: str):
        super().__init__()
        self.kind = spec["type"]
        self.norm1 = _fp32_param((width,))
        self.mixer = make_mixer(self.kind, spec["mixer"], width, eps, quant_config, f"{prefix}.mixer")
        self.has_mlp = spec.get("mlp") is not None
        self.ls1 = _fp32_param((width,))
        # one GEMM for the gates of both sub-layers: they read the same h
        self.gates = MergedColumnParallelLinear(width, [width] * (2 if self.has_mlp else 1), bias=True,
                                                quant_config=quant_config, prefix=f"{prefix}.gates")
        if self.has_mlp:
            self.ls2 = _fp32_param((width,))
            self.mlp = LefolornMoE(width, spec["mlp"], quant_config, f"{prefix}.mlp")

    def forward(self, x: torch.Tensor, h: torch.Tensor, positions: torch.Tensor, lent: dict,
                next_norm: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
        """``x``: the fp32 residual, updated in place; ``h``: this layer's normed input; returns the next layer's."""
        W = x.shape[1]
        y = self.mixer(h, positions, 0, lent) if self.kind != "latent_attention" else self.mixer(h, positions)
        g = self.gates(h)
        subs = [(y, self.ls1, g[:, :W], None, None)]
        if self.has_mlp:
            f, shared, idw = self.mlp(h)
            subs.append((f, self.ls2, g[:, W:], h if idw is not None else None, idw))
            if shared is not None:              # joins inside the same pass, behind the feed-forward's scale and gate
                subs.append((shared, self.ls2, g[:, W:], None, None))
        return ops.gated_residual_group_norm(x, subs, next_norm, groups, eps, h.dtype)


class LefolornForCausalLM(nn.Module):
    supports_pp = False
    supports_lora = False
    # kernels outside the common set that this model launches (ops/build.py builds them on first use)
    native_sources = ("masked_attention.hip", "attention.hip", "attention_prefill.hip", "latent_attention.hip",
                      "mla.hip", "moe.hip", "gemm_tile.hip")

    def __init__(self, vllm_config: VllmConfig, prefix: str = ""):
        super().__init__()
        config = vllm_config.model_config.hf_config
        self.config = config
        quant_config = getattr(vllm_config, "quant_config", None)
        width, self.eps = int(config.width), float(config.norm["eps"])
        self.groups = int(config.norm.get("groups", 1) or 1)
        if width % self.groups:
            raise ValueError(f"a width of {width} does not split into {self.groups} equal parts")
        mixing = [i for i, l in enumerate(config.layers) if l["type"] != "latent_attention" and l["mixer"].get("v_mix")]
        rows = {int(config.layers[i]["mixer"]["kv_heads"]) * int(config.layers[i]["mixer"]["vdim"]) for i in mixing}
        if len(rows) > 1:
            raise ValueError(f"layers {mixing} mix their values but make rows of different widths {sorted(rows)}")
        self.embed_tokens = VocabParallelEmbedding(int(config.vocab), width)
        self.layers = nn.ModuleList([LefolornLayer(spec, width, self.eps, quant_config, f"layers.{i}")
                                     for i, spec in enumerate(config.layers)])
        self.norm = _fp32_param((width,))
        self.lm_head = ParallelLMHead(int(config.vocab), width)
        self.logits_processor = LogitsProcessor(int(config.vocab))

    def get_input_embeddings(self, input_ids):
        return self.embed_tokens(input_ids)

    def forward(self, input_ids, positions, intermediate_tensors=None, inputs_embeds=None):
        e = inputs_embeds if inputs_embeds is not None else self.embed_tokens(input_ids)
        dtype = self.embed_tokens.weight.dtype
        x = e.float().contiguous() if e.dtype != torch.float32 else e.clone()
        norms = [l.norm1 for l in self.layers] + [self.norm]
        h = ops.gated_residual_group_norm(x, [], norms[0], self.groups, self.eps, dtype)
        lent: dict = {}                 # what layers of this pass hand to later ones (the first mixed values)
        for i, layer in enumerate(self.layers):
            h = layer(x, h, positions, lent, norms[i + 1], self.groups, self.eps)
        return h

    def compute_logits(self, hidden_states):
        return self.logits_processor(self.lm_head, hidden_states).float()

    # checkpoint name -> (parameter name, shard id)
    _MIX = {
        "attention": {"q": ("in_proj.weight", 0), "k": ("in_proj.weight", 1), "v": ("in_proj.weight", 2),
                      "q.b": ("in_proj.bias", 0), "k.b": ("in_proj.bias", 1), "v.b": ("in_proj.bias", 2),
                      "g": ("in_proj.weight", 3), "q.norm": ("q_norm", None), "k.norm": ("k_norm", None),
                      "rel": ("rel", None), "vmix": ("vmix", None), "o": ("o_proj.weight", None)},
        "latent_attention": {"dq": ("down_proj.weight", 0), "dkv": ("down_proj.weight", 1),
                             "dq.norm": ("q_norm", None), "uq": ("uq_proj.weight", None),
                             "dkv.norm": ("c_norm", None), "uk": ("uk_proj.weight", None),
                             "uv": ("uv_proj.weight", None), "sink": ("sink", None), "o": ("o_proj.weight", None)},
    }
    _MIX["attention_2"] = {k: v for k, v in _MIX["attention"].items() if k not in ("g", "rel")}
    _FF = {"gate": ("gate_up_proj.weight", 0), "up": ("gate_up_proj.weight", 1), "down": ("down_proj.weight", None)}
    _TOP = {"embed": "embed_tokens.weight", "head": "lm_head.weight", "final.norm": "norm"}
    _EXPERT = {"gate": ("w13_weight", "w1"), "up": ("w13_weight", "w3"), "down": ("w2_weight", "w2")}
    _LAYER = {"norm1": ("norm1", None), "ls1": ("ls1", None), "ls2": ("ls2", None), "rg1": ("gates.weight", 0),
              "rg1.b": ("gates.bias", 0), "rg2": ("gates.weight", 1), "rg2.b": ("gates.bias", 1)}
    _FF_ONLY = ("ls2", "rg2", "rg2.b")

    def _target(self, name: str):
        """Returns (parameter name, shard id, expert id) or None."""
        if name in self._TOP:
            return self._TOP[name], None, None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None
        i, rest = int(m.group(1)), m.group(2)
        layer, base = self.layers[i], f"layers.{i}."
        if rest in self._LAYER:
            t, shard = self._LAYER[rest]
            if rest in self._FF_ONLY and not layer.has_mlp:
                return base + "no_feed_forward." + rest, None, None
            return base + t, shard, None
        part, _, leaf = rest.partition(".")
        if part == "mix" and leaf in self._MIX[layer.kind]:
            t, shard = self._MIX[layer.kind][leaf]
            return f"{base}mixer.{t}", shard, None
        if part == "mlp" and layer.has_mlp:
            if leaf == "router":
                return f"{base}mlp.router_weight", None, None
            if leaf == "correction":
                return f"{base}mlp.correction", None, None
            sub, _, w = leaf.partition(".")
            if sub == "shared" and layer.mlp.shared is not None and w in self._FF:
                t, shard = self._FF[w]
                return f"{base}mlp.shared.{t}", shard, None
            em = re.fullmatch(r"e(\d+)", sub)
            if em and w in self._EXPERT and int(em.group(1)) < layer.mlp.experts.global_num_experts:
                t, shard = self._EXPERT[w]
                return f"{base}mlp.experts.{t}", shard, int(em.group(1))
        return None

    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> set[str]:
        params = dict(self.named_parameters())
        loaded: set[str] = set()
        for name, t in weights:
            tgt = self._target(name)
            if tgt is None:
                raise ValueError(f"checkpoint tensor {name!r} has no place in this model")
            target, shard, expert = tgt
            if target not in params:
                # tensors the design never reads: the value-mixing weight of a layer that lends its values or does not
                # mix, the feed-forward's scale and gate of a layer without a feed-forward
                if name.endswith((".mix.vmix", ".ls2", ".rg2", ".rg2.b")):
                    continue
                raise ValueError(f"checkpoint tensor {name!r} has no place in this model")
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
