"""Latent attention over a sliding window: keys and values are up-projections of one low-rank latent per token,
plus a rotated key part that all heads share; only the latent and that part are cached.

    q = W_q x                      per head [D plain | P rotated]; with ``q_rank``: q = W_uq (W_dq x / rms * q_norm), the
                                   queries through a normed latent of their own
    [c_raw | k_rot] = W_dkv x      c = c_raw / rms(c_raw) * c_norm  (R values);  k_rot: P values, rotated, no norm
    k_h = W_uk_h c,  v_h = W_uv_h c
    score(i, j, h) = scale * (q_plain . k_h + q_rot . k_rot),   j <= i and i - j < window,   softmax over j
                                   (``sink``: a learned number per head whose exponential joins the denominator)
    out = W_o [sum_j p v_h]_h

The rotation turns the pairs (2i, 2i + 1), i < rot_dims / 2, of the P rotated values by position * base^(-2i / rot_dims)
(angles, cosines and sines in fp32; values past rot_dims pass unchanged).  The key up-projection is folded into the
query (q_abs = W_uk_h^T q_plain, so the score is q_abs . c + q_rot . k_rot) and the value up-projection is applied
after the attention, which then runs over the cached rows [c | k_rot] for all heads alike: the cache holds R + P
values per token (``MLAAttention``; the MFMA kernel keeps a transposed copy of c beside them).  A mixer whose weights serve several passes of a looped
stack owns one cache per pass.
Kernels: ops/csrc/latent_attention.hip.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import envs, ops
from ..config import get_current_vllm_config
from ..forward_context import get_forward_context
from ..parallel.state import get_tensor_model_parallel_world_size
from .attention import MLAAttention
from .hyper_connections import _fp32_param
from .linear import MergedColumnParallelLinear, ReplicatedLinear, RowParallelLinear

_TABLES: dict = {}


def interleaved_cos_sin(max_len: int, dims: int, base: float, device) -> torch.Tensor:
    """fp32 [max_len, dims]: cos(p * f_i) for i < dims / 2, then sin(p * f_i), f_i = base^(-2i / dims)."""
    key = (int(max_len), int(dims), float(base), str(device))
    t = _TABLES.get(key)
    if t is None and dims == 0:
        t = _TABLES[key] = torch.zeros((max_len, 1), dtype=torch.float32, device=device)
    if t is None:
        i = torch.arange(dims // 2, dtype=torch.float32, device=device)
        f = float(base) ** (-2.0 * i / float(dims))
        ang = torch.arange(max_len, dtype=torch.float32, device=device)[:, None] * f[None, :]
        t = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1).contiguous()
        _TABLES[key] = t
    return t


class WindowedLatentAttention(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, kv_rank: int,
                 scale: float, window: Optional[int], rot_base: Optional[float], rot_dims: int, eps: float,
                 passes: int = 1, quant_config=None, prefix: str = "", q_rank: int = 0, sink: bool = False):
        super().__init__()
        if get_tensor_model_parallel_world_size() > 1:
            raise NotImplementedError("windowed latent attention runs with tensor_parallel_size=1")
        H, D, P, Dv, R = int(num_heads), int(head_dim), int(rot_dim), int(v_head_dim), int(kv_rank)
        self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank = H, D, P, Dv, R
        self.eps = float(eps)
        self.rot_dims = int(rot_dims) if rot_base else 0
        if self.rot_dims > P or self.rot_dims % 2:
            raise ValueError(f"{prefix}: {self.rot_dims} rotated dimensions do not fit an even part of {P}")
        self.q_rank = int(q_rank or 0)
        if self.q_rank:
            # one GEMM for both down-projections: [query latent | key / value latent + rotated key part]
            self.down_proj = MergedColumnParallelLinear(hidden_size, [self.q_rank, R + P], bias=False,
                                                        quant_config=quant_config, prefix=f"{prefix}.down_proj")
            self.q_norm = _fp32_param((self.q_rank,))
            self.uq_proj = ReplicatedLinear(self.q_rank, H * (D + P), bias=False, quant_config=quant_config,
                                            prefix=f"{prefix}.uq_proj")
        else:
            self.q_proj = ReplicatedLinear(hidden_size, H * (D + P), bias=False, quant_config=quant_config,
                                           prefix=f"{prefix}.q_proj")
            self.dkv_proj = ReplicatedLinear(hidden_size, R + P, bias=False, quant_config=quant_config,
                                             prefix=f"{prefix}.dkv_proj")
        self.sink = _fp32_param((H,), 0.0) if sink else None
        self.uk_proj = ReplicatedLinear(R, H * D, bias=False, prefix=f"{prefix}.uk_proj")
        self.uv_proj = ReplicatedLinear(R, H * Dv, bias=False, prefix=f"{prefix}.uv_proj")
        self.o_proj = RowParallelLinear(H * Dv, hidden_size, bias=False, quant_config=quant_config,
                                        prefix=f"{prefix}.o_proj")
        self.c_norm = _fp32_param((R,))
        cfg = get_current_vllm_config()
        # 16-bit activations and sizes the MFMA kernel is built for: that kernel (it wants a transposed copy of the
        # latent beside the rows); anything else, fp32 included: the kernel for any sizes on the rows alone
        self.use_mfma = bool(cfg.device_config.device != "cpu" and not envs.VDA_FORCE_TORCH_OPS and envs.VDA_MLA
                             and cfg.model_config.dtype in (torch.bfloat16, torch.float16)
                             and cfg.cache_config.cache_dtype == "auto" and (R + P, R) in ops.MLA_KERNEL_SIZES)
        self.attn = nn.ModuleList([
            MLAAttention(H, R, P, float(scale), prefix=f"{prefix}.attn.{i}", sliding_window=int(window or 0),
                         transposed_copy=self.use_mfma) for i in range(passes)])
        self.max_len = int(cfg.model_config.max_model_len) + 1
        self.rot_base = float(rot_base) if rot_base else 0.0
        self._cos_sin: Optional[torch.Tensor] = None
        self._w_uk = self._w_uv_t = None

    def _tables(self, device) -> torch.Tensor:
        if self._cos_sin is None or self._cos_sin.device != device:
            self._cos_sin = interleaved_cos_sin(self.max_len, self.rot_dims, self.rot_base or 1.0, device)
        return self._cos_sin

    def _folded_weights(self):
        """W_uk as [H, D, R] (a view) and W_uv^T as [H, R, Dv] (a copy made once)."""
        w = self.uk_proj.weight
        if self._w_uk is None or self._w_uk.data_ptr() != w.data_ptr():
            self._w_uk = w.view(self.num_heads, self.head_dim, self.kv_rank)
            self._w_uv_t = self.uv_proj.weight.view(self.num_heads, self.v_head_dim, self.kv_rank) \
                .transpose(1, 2).contiguous()
        return self._w_uk, self._w_uv_t

    def forward(self, x: torch.Tensor, positions: torch.Tensor, pass_index: int = 0) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        attn = self.attn[pass_index]
        H, D, P, Dv, R = self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank
        T = x.shape[0]
        if self.q_rank:
            both = self.down_proj(x)
            q = self.uq_proj(ops.group_rms_norm(both[:, : self.q_rank], self.q_norm, self.eps, 1))
            down = both[:, self.q_rank:]
        else:
            q = self.q_proj(x)
            down = self.dkv_proj(x)
        w_uk, w_uv_t = self._folded_weights()
        qf = torch.empty((T, H, R + P), dtype=q.dtype, device=q.device)
        q3 = q.view(T, H, D + P)
        # q_abs[t, h] = W_uk_h^T q_plain[t, h]: one batched product over the heads
        torch.bmm(q3[:, :, :D].transpose(0, 1), w_uk, out=qf[:, :, :R].transpose(0, 1))
        if md is None or attn.k_cache is None:           # memory-profiling run: the projections carry the footprint
            qf[:, :, R:] = q3[:, :, D:]
            o_lat = qf[:, :, :R] + down[:, None, :R]
        else:
            n = md.num_actual_tokens
            if n < T:
                qf[n:, :, R:].zero_()
            ops.latent_norm_rope_cache(q[:n], down[:n], self.c_norm, self._tables(q.device), positions[:n], qf[:n],
                                       attn.k_cache, md.slot_mapping[:n], H, D, P, R, self.rot_dims, self.eps,
                                       attn.v_cache if self.use_mfma else None)
            o_lat = attn.forward_cached(qf, self.sink)
        o = torch.bmm(o_lat.transpose(0, 1), w_uv_t).transpose(0, 1)
        return self.o_proj(o.reshape(T, H * Dv))
