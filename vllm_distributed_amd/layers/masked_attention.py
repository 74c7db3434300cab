"""Softmax attention assembled from options: per-head query / key norms, part-rotated heads, a short causal convolution
on the projections, several score maps per head, window / chunk masks, sinks and an output gate.

    q, k, v = W x + b                                   (optional biases; grouped query heads; key width D, value width Dv)
    q, k, v <- causal convolution over time, per channel (``conv_taps`` >= 1; no bias, no activation; one tap is a
               weight per channel)
    q, k    <- q / rms(q) * q_norm, k / rms(k) * k_norm  per head and map (weights of size D shared by all heads)
    q, k    <- first ``rot_dims`` values of each map rotated, value i paired with i + rot_dims / 2 (``rot_pairing``
               "halves") or value 2i with 2i + 1 ("neighbours"), fp32 angles
    q       <- q * (1 + coef * ln(floor((p + 1) / every) + 1)) at position p (``q_temp`` = (coef, every))
    v       <- (1 - lam) v + lam v_first (``v_mix``): v_first are the values that the first such layer of the stack
               made of the same token; the layers of one forward pass hand them on through a dictionary
    score   = scale * q . k;  score <- cap * tanh(score / cap) (``softcap``);  score += rel[bucket(i - j), h]
               (``dist_bias`` = (rows, far): distances below rows / 2 have a row each, the others share the rest in
               logarithmic steps up to ``far``)
    key j visible to query i: j <= i, i - j < window, j // chunk == i // chunk
    softmax over the visible keys; with ``sink`` the denominator also holds exp(sink[h]) (a learned number per head),
               with ``sink_fixed`` = s it holds exp(s) (s = 0: one more 1)
    maps == 2 (differential attention): a head's query / key rows hold two maps side by side, each an attention over
               the same values;  o = a1 - lam * a2,  lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff,
               then o / rms(o) * (1 - diff) over the head's Dv values
    out     = W_o (o * sigmoid(W_g x))                   (``gate``)

The layer owns pages of the ordinary paged KV cache (a full-attention layer to the scheduler and the KV-cache manager:
keys that a window or chunk hides stay in their pages, the kernels never load them) and, with a convolution, a state
slot per request for the last ``conv_taps - 1`` projected rows (the slots of the recurrent mixers).  A stack that runs
one set of weights at several depths gives every use a cache and state of its own (``users``).
Cache layout: K [blocks, G, block, maps * D] (normed and rotated), V [blocks, G, Dv, block].
With 16-bit activations and keys and values of one width that the matrix-core paged attention kernels are built for,
those kernels run (ops/csrc/attention.hip with the window, chunk and sink as options); every score map is then a key
head of its own in the cache, K [blocks, G * maps, block, D] in the same memory, and an epilogue kernel combines the maps.
Kernels: ops/csrc/masked_attention.hip, ops/csrc/attention.hip, ops/csrc/mamba.hip (the convolution shared with the
state-space mixers).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..config import get_current_vllm_config
from ..forward_context import get_forward_context
from ..models.mamba import StateSpaceLayer
from ..parallel.state import get_tensor_model_parallel_world_size
from ..sched.kv_cache_interface import FullAttentionSpec, KVCacheSpec
from .hyper_connections import _fp32_param
from .linear import MergedColumnParallelLinear, RowParallelLinear, set_weight_attrs
from .rotary import half_split_cos_sin


def log_bucket_rows(rows: int, far: int) -> torch.Tensor:
    """Row of a distance table for every distance 0 .. far: n itself below rows / 2, then
    min(rows - 1, rows / 2 + floor(ln(n / (rows / 2)) / ln(far / (rows / 2)) * (rows - rows / 2)));
    ``far`` and everything beyond share the last row.  int64 [far + 1]."""
    import math
    half = rows // 2
    out = []
    for n in range(int(far) + 1):
        if n < half or half == 0:
            out.append(min(n, rows - 1))
        else:
            out.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))))
    return torch.tensor(out, dtype=torch.int64)


class PagedKV(nn.Module):
    """The pages of one use of an attention mixer's weights."""
    is_paged_kv_layer = True

    def __init__(self, num_kv_heads: int, k_row: int, v_head_dim: int, prefix: str = ""):
        super().__init__()
        self.num_kv_heads, self.k_row, self.v_head_dim = num_kv_heads, k_row, v_head_dim
        self.layer_name = prefix
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None

    def get_kv_cache_spec(self, block_size: int, dtype: torch.dtype) -> KVCacheSpec:
        return FullAttentionSpec(block_size=block_size, num_kv_heads=self.num_kv_heads, head_size=self.k_row,
                                 dtype=dtype, v_head_size=self.v_head_dim)

    def bind_kv_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
        self.k_cache, self.v_cache = k_cache, v_cache


class ShortConvState(StateSpaceLayer):
    """The last ``taps - 1`` rows that entered a short causal convolution, per request."""

    def __init__(self, channels: int, taps: int, prefix: str = ""):
        super().__init__()
        self.channels, self.taps = int(channels), int(taps)
        self.conv_dtype = torch.get_default_dtype()
        self.state_dtypes = (self.conv_dtype, torch.float32)
        self.layer_name = prefix

    def state_shapes(self) -> tuple:
        return ((self.channels, self.taps - 1), (4,))          # no recurrent part: a 16-byte placeholder


class MaskedSoftmaxAttention(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, eps: float, *, bias: bool = False, conv_taps: int = 0, window: int = 0, chunk: int = 0,
                 sink: bool = False, maps: int = 1, diff: float = 0.0, gate: bool = False, rot_dims: int = 0,
                 rot_base: float = 10000.0, rot_scaling: Optional[dict] = None, users: int = 1, quant_config=None,
                 prefix: str = "", rot_pairing: str = "halves", q_temp: Optional[tuple] = None, softcap: float = 0.0,
                 dist_bias: Optional[tuple] = None, sink_fixed: Optional[float] = None, v_mix: bool = False):
        super().__init__()
        if get_tensor_model_parallel_world_size() > 1:
            raise NotImplementedError("this attention layer runs with tensor_parallel_size=1")
        H, G, D, Dv = int(num_heads), int(num_kv_heads), int(head_dim), int(v_head_dim)
        if H % G:
            raise ValueError(f"{prefix}: {H} query heads do not divide into {G} key/value heads")
        if maps not in (1, 2):
            raise ValueError(f"{prefix}: {maps} score maps per head (1 or 2)")
        if rot_dims % 2 or rot_dims > D:
            raise ValueError(f"{prefix}: {rot_dims} rotated dimensions do not fit an even part of {D}")
        self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim = H, G, D, Dv
        self.scale, self.eps = float(scale), float(eps)
        self.window, self.chunk, self.maps, self.diff = int(window or 0), int(chunk or 0), int(maps), float(diff)
        self.taps = int(conv_taps or 0)
        self.rot_dims, self.rot_base, self.rot_scaling = int(rot_dims), float(rot_base), rot_scaling
        if rot_pairing not in ("halves", "neighbours") or (rot_pairing == "neighbours" and rot_scaling):
            raise ValueError(f"{prefix}: rotation pairing {rot_pairing!r} (with frequency scaling: halves only)")
        if sink and sink_fixed is not None:
            raise ValueError(f"{prefix}: a learned sink and a fixed one exclude each other")
        self.rot_pairing = rot_pairing
        self.q_temp = (float(q_temp[0]), int(q_temp[1])) if q_temp else None
        if self.q_temp and self.q_temp[1] < 1:
            raise ValueError(f"{prefix}: the query temperature grows every {self.q_temp[1]} positions")
        self.softcap = float(softcap or 0.0)
        self.layer_name = prefix
        nq, nk, nv = H * maps * D, G * maps * D, G * Dv
        self.qkv_width = nq + nk + nv
        sizes = [nq, nk, nv] + ([H * Dv] if gate else [])
        # one GEMM for everything that reads x: q | k | v (| gate); the gate's part of the bias stays zero
        self.in_proj = MergedColumnParallelLinear(hidden_size, sizes, bias=bias, quant_config=quant_config,
                                                  prefix=f"{prefix}.in_proj")
        self.has_gate = bool(gate)
        self.o_proj = RowParallelLinear(H * Dv, hidden_size, bias=False, quant_config=quant_config,
                                        prefix=f"{prefix}.o_proj")
        self.q_norm = _fp32_param((D,))
        self.k_norm = _fp32_param((D,))
        if sink_fixed is not None:
            self.register_buffer("sink", torch.full((H,), float(sink_fixed), dtype=torch.float32), persistent=False)
        else:
            self.sink = _fp32_param((H,), 0.0) if sink else None
        # learned bias per (distance bucket, head); the kernels read one row per distance, made once after loading
        self.dist_far = 0
        if dist_bias:
            rows, self.dist_far = int(dist_bias[0]), int(dist_bias[1])
            if rows < 2 or self.dist_far <= rows // 2:
                raise ValueError(f"{prefix}: {rows} distance buckets up to {self.dist_far}")
            self.rel = _fp32_param((rows, H), 0.0)
            self.register_buffer("_bucket", log_bucket_rows(rows, self.dist_far), persistent=False)
        self._dist_table: Optional[torch.Tensor] = None
        self.vmix = _fp32_param((1,), 0.0) if v_mix else None
        if maps == 2:
            self.lq1, self.lk1 = _fp32_param((D,), 0.0), _fp32_param((D,), 0.0)
            self.lq2, self.lk2 = _fp32_param((D,), 0.0), _fp32_param((D,), 0.0)
        self._lam: Optional[torch.Tensor] = None
        if self.taps >= 1:
            dtype = torch.get_default_dtype()
            self.conv_weight = nn.Parameter(torch.zeros((self.qkv_width, self.taps), dtype=dtype), requires_grad=False)
            offs = [0, nq, nq + nk]

            def load_conv(param, t, shard_id=None):
                if shard_id is None:
                    param.data.copy_(t.reshape(param.shape))
                else:
                    t = t.reshape(t.shape[0], -1)
                    param.data[offs[shard_id]: offs[shard_id] + t.shape[0]].copy_(t)
            set_weight_attrs(self.conv_weight, {"weight_loader": load_conv})
            # one tap: a weight per channel, no earlier rows, nothing carried
            self.conv_states = nn.ModuleList([ShortConvState(self.qkv_width, self.taps, f"{prefix}.conv.{i}")
                                              for i in range(users if self.taps > 1 else 0)])
        self.caches = nn.ModuleList([PagedKV(G, maps * D, Dv, f"{prefix}.kv.{i}") for i in range(users)])
        cfg = get_current_vllm_config()
        # 16-bit activations and head widths the matrix-core paged attention kernels are built for: those kernels (every
        # score map a key head of its own in the cache); anything else, fp32 included: the kernel for any sizes
        self.use_mfma = ops.masked_attention_mfma_ok(H, G, D, Dv, maps, self.sink is not None, cfg.model_config.dtype,
                                                     cfg.device_config.device != "cpu") \
            and cfg.cache_config.cache_dtype == "auto" and not (self.dist_far and maps == 2)
        self.max_len = int(cfg.model_config.max_model_len) + 1
        self._cos_sin: Optional[torch.Tensor] = None

    def _table(self, device) -> Optional[torch.Tensor]:
        if self.rot_dims == 0:
            return None
        if self._cos_sin is None or self._cos_sin.device != device:
            if self.rot_pairing == "neighbours":
                from .latent_attention import interleaved_cos_sin
                self._cos_sin = interleaved_cos_sin(self.max_len, self.rot_dims, self.rot_base, device)
            else:
                self._cos_sin = half_split_cos_sin(self.max_len, self.rot_dims, self.rot_base, self.rot_scaling,
                                                   device)
        return self._cos_sin

    def _distances(self) -> Optional[torch.Tensor]:
        """fp32 [far + 1, H]: the bias of every distance, the learned rows spread over their buckets (made once from
        the loaded table); for the matrix-core kernels one padded row per head instead."""
        if not self.dist_far:
            return None
        if self._dist_table is None or self._dist_table.device != self.rel.device:
            self._dist_table = self.rel.data[self._bucket.to(self.rel.device)].contiguous()
            if self.use_mfma:             # one padded row per head
                self._dist_table = ops.padded_distance_rows(self._dist_table)
        return self._dist_table

    def _lambda(self) -> Optional[torch.Tensor]:
        """The weight of the second map, one fp32 value on the device (made once from the loaded vectors)."""
        if self.maps != 2:
            return None
        if self._lam is None or self._lam.device != self.lq1.device:
            self._lam = (torch.exp((self.lq1 * self.lk1).sum()) - torch.exp((self.lq2 * self.lk2).sum())
                         + self.diff).reshape(1).contiguous()
        return self._lam

    def forward(self, x: torch.Tensor, positions: torch.Tensor, user: int = 0,
                lent: Optional[dict] = None) -> torch.Tensor:
        """``lent``: a dictionary that lives for one forward pass of the stack; the first layer with ``v_mix`` puts its
        values there ("v_first") and the later ones mix them into their own."""
        md = get_forward_context().attn_metadata
        H, G, D, Dv, maps = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, self.maps
        kv = self.caches[user]
        p = self.in_proj(x)
        T = p.shape[0]
        W = self.qkv_width
        gate = p[:, W:] if self.has_gate else None
        if md is None or kv.k_cache is None:              # memory-profiling run: the projections carry the footprint
            o = p[:, : H * maps * D].reshape(T, H, maps * D)[..., :1].expand(T, H, Dv).reshape(T, H * Dv)
            return self.o_proj((o * gate if gate is not None else o).contiguous())
        n = md.num_actual_tokens
        S = md.num_decode_seqs + md.num_prefill_seqs
        qsl, lens = md.query_start_loc[:S + 1], md.seq_lens[:S]
        qkv = p[:n]
        if self.taps > 1:
            st = self.conv_states[user]
            tbl = StateSpaceLayer.slot_table(md)[:S]
            qkv = ops.causal_conv1d(p[:n, :W], self.conv_weight, None, st.conv_state, qsl, lens, tbl,
                                    md.max_query_len, activation=False)
        elif self.taps == 1:
            qkv = (p[:n, :W].float() * self.conv_weight.float().view(1, -1)).to(p.dtype)
        g_rows = gate[:n] if gate is not None else None
        extras = dict(pairing=self.rot_pairing, q_temp=self.q_temp)
        if self.vmix is not None:
            if lent is None:
                raise ValueError(f"{self.layer_name}: value mixing needs the forward pass's dictionary")
            if "v_first" in lent:
                extras.update(v_first=lent["v_first"], v_lam=self.vmix)
            else:
                lent["v_first"] = qkv[:, (H + G) * maps * D: (H + G) * maps * D + G * Dv]
        if self.use_mfma:
            qn = ops.qk_norm_rope_cache(qkv, H, G, D, Dv, maps, self.q_norm, self.k_norm, self._table(p.device),
                                        positions[:n], self.rot_dims, self.eps, kv.k_cache, kv.v_cache,
                                        md.slot_mapping[:n], by_map=True, **extras)
            nd, ndt, n_pre, npt, pqsl = (md.num_decode_seqs, md.num_decode_tokens, md.num_prefill_seqs,
                                         md.num_prefill_tokens, md.prefill_query_start_loc)
            cols = max(md.max_decode_query_len, 1) * (H // G)
            if nd > 0 and (cols > 32 or (cols > 16 and D > 128)):
                # more query rows per key head than the decode form takes: the tiled form serves every sequence
                nd, ndt, n_pre, npt, pqsl = 0, 0, S, n, qsl
            out = ops.masked_softmax_attention_mfma(
                qn, kv.k_cache, kv.v_cache, md.block_table, md.seq_lens, md.query_start_loc, pqsl, nd, ndt, n_pre, npt,
                md.max_decode_query_len, md.decode_num_splits, md.max_query_len, self.scale, H, self.window,
                self.chunk, self.sink, maps, self._lambda(), self.eps, 1.0 - self.diff, g_rows,
                softcap=self.softcap, dist_bias=self._distances())
            if n < T:
                out = torch.cat([out, out.new_zeros((T - n, out.shape[1]))], dim=0)
            return self.o_proj(out)
        qn = ops.qk_norm_rope_cache(qkv, H, G, D, Dv, maps, self.q_norm, self.k_norm, self._table(p.device),
                                    positions[:n], self.rot_dims, self.eps, kv.k_cache, kv.v_cache,
                                    md.slot_mapping[:n], **extras)
        out = ops.masked_softmax_attention(qn, kv.k_cache, kv.v_cache, md.block_table[:S], lens, qsl, self.scale,
                                           self.window, self.chunk, self.sink, maps, self._lambda(), self.eps,
                                           1.0 - self.diff, gate[:n] if gate is not None else None,
                                           md.max_query_len, p.dtype, softcap=self.softcap,
                                           dist_bias=self._distances())
        if n < T:
            out = torch.cat([out, out.new_zeros((T - n, out.shape[1]))], dim=0)
        return self.o_proj(out)
