"""Plain PyTorch implementations of every op in this package.

They serve two purposes: (1) the numerics oracle the HIP kernels are tested
against (fp32 math, same layouts), and (2) the CPU plumbing path used when no
GPU is present (role of the reference's csrc/cpu backend for the OPT-125m CPU
configuration).  They are never used for CUDA tensors unless
``VDA_FORCE_TORCH_OPS=1`` is set for debugging.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F

FP8_MAX = 448.0


# ---- norms -----------------------------------------------------------------
def rms_norm(x, weight, eps, residual=None, weight_bias: float = 0.0):
    dt = x.dtype
    if residual is not None:
        x = (x.float() + residual.float()).to(dt)
        residual.copy_(x)
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    y = (xf * torch.rsqrt(var + eps)).to(dt)
    return (y.float() * (weight.float() + weight_bias)).to(dt)


def layer_norm(x, weight, bias, eps):
    return F.layer_norm(x.float(), (x.shape[-1],), weight.float(),
                        None if bias is None else bias.float(), eps).to(x.dtype)


# ---- activations -------------------------------------------------------------
def _act(kind: str, x: torch.Tensor, threshold: float = 0.0) -> torch.Tensor:
    if kind == "silu":
        return F.silu(x)
    if kind == "gelu":
        return F.gelu(x)
    if kind in ("gelu_tanh", "gelu_pytorch_tanh", "gelu_new"):
        return F.gelu(x, approximate="tanh")
    if kind == "relu":
        return F.relu(x)
    if kind == "gelu_fast":
        return 0.5 * x * (1.0 + torch.tanh(x * 0.79788456 * (1.0 + 0.044715 * x * x)))
    if kind in ("quick_gelu", "gelu_quick"):
        return x * torch.sigmoid(1.702 * x)
    if kind == "fatrelu":
        return torch.where(x > threshold, x, torch.zeros_like(x))
    if kind == "relu2":
        return F.relu(x).square()
    raise ValueError(f"unknown activation {kind!r}")


def clamped_swiglu(g, u, limit: float):
    """min(g, limit) * sigmoid(1.702 min(g, limit)) * (clamp(u, -limit, limit) + 1)."""
    g = g.clamp(max=limit)
    return g * torch.sigmoid(1.702 * g) * (u.clamp(-limit, limit) + 1.0)


def act_and_mul(x, kind="silu", act_first=True, threshold=0.0):
    d = x.shape[-1] // 2
    a, b = x[..., :d].float(), x[..., d:].float()
    if kind == "clamped_swiglu":          # ``threshold`` carries the limit
        return clamped_swiglu(a, b, threshold).to(x.dtype)
    y = _act(kind, a, threshold) * b if act_first else a * _act(kind, b, threshold)
    return y.to(x.dtype)


def activation(x, kind, threshold=0.0):
    return _act(kind, x.float(), threshold).to(x.dtype)


# ---- rotary ------------------------------------------------------------------
def _rotate(x, cos, sin, rot_dim, is_neox):
    # x: [T, H, D]; cos/sin: [T, rot_dim/2]
    xr = x[..., :rot_dim].float()
    cos, sin = cos[:, None, :], sin[:, None, :]
    if is_neox:
        x1, x2 = xr[..., : rot_dim // 2], xr[..., rot_dim // 2:]
        out = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)
    else:
        x1, x2 = xr[..., 0::2], xr[..., 1::2]
        out = torch.stack((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).flatten(-2)
    res = x.clone()
    res[..., :rot_dim] = out.to(x.dtype)
    return res


def rotary_embedding(positions, q, k, cos_sin_cache, rot_dim, head_size, is_neox=True):
    """In place on q [T, Hq*D] / k [T, Hkv*D] (k may be None)."""
    cs = cos_sin_cache[positions.long()]
    cos, sin = cs[:, : rot_dim // 2].float(), cs[:, rot_dim // 2:].float()
    T = q.shape[0]
    qv = q.view(T, -1, head_size)
    qv.copy_(_rotate(qv, cos, sin, rot_dim, is_neox))
    if k is not None:
        kv = k.view(T, -1, head_size)
        kv.copy_(_rotate(kv, cos, sin, rot_dim, is_neox))


# ---- cache ---------------------------------------------------------------------
def reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, k_scale: float = 1.0, v_scale: float = 1.0):
    """k, v: [T, Hkv, D]; k_cache [nblk, Hkv, BS, D]; v_cache [nblk, Hkv, D, BS]; fp8 caches hold x / scale."""
    bs = k_cache.shape[2]
    slots = slot_mapping.long()
    keep = slots >= 0
    slots = slots[keep]
    blk, off = slots // bs, slots % bs
    kk, vv = k[keep], v[keep]
    if k_cache.dtype == torch.float8_e4m3fn:
        kk = (kk.float() / k_scale).clamp(-448, 448)
        vv = (vv.float() / v_scale).clamp(-448, 448)
    k_cache[blk, :, off, :] = kk.to(k_cache.dtype)
    v_cache[blk, :, :, off] = vv.to(v_cache.dtype)


def gather_cache(k_cache, v_cache, slots):
    bs = k_cache.shape[2]
    slots = slots.long()
    blk, off = slots // bs, slots % bs
    return k_cache[blk, :, off, :], v_cache[blk, :, :, off]


def copy_blocks(cache, pairs):
    for s, d in pairs.tolist():
        cache[d].copy_(cache[s])


def transfer_blocks(dst, src, dst_ids, src_ids):
    dst[dst_ids.long().to(dst.device)] = src[src_ids.long().to(src.device)].to(dst.device)


# ---- attention -------------------------------------------------------------------
def paged_attention(q, k_cache, v_cache, block_table, seq_lens, q_start_loc, scale,
                    window: int = 0, softcap: float = 0.0, alibi=None, return_lse: bool = False,
                    k_scale: float = 1.0, v_scale: float = 1.0, causal: bool = True, visible=None):
    """Attention of the new tokens of every sequence against its paged K/V (which already contain
    the new tokens); causal, or over every key of the sequence.  q: [T, Hq, D] -> [T, Hq, D].
    ``visible(pos [ql, 1], key [1, sl]) -> bool [Hq, ql, sl]``: an extra per-head visibility pattern."""
    T, Hq, D = q.shape
    Hkv, bs = k_cache.shape[1], k_cache.shape[2]
    G = Hq // Hkv
    out = torch.zeros_like(q)
    lse = torch.full((Hq, T), float("-inf"), dtype=torch.float32, device=q.device)
    qsl = q_start_loc.tolist()
    for s, sl in enumerate(seq_lens.tolist()):
        a, b = qsl[s], qsl[s + 1]
        ql = b - a
        if ql == 0 or sl == 0:
            continue
        nb = (sl + bs - 1) // bs
        blocks = block_table[s, :nb].long()
        k = k_cache[blocks].permute(1, 0, 2, 3).reshape(Hkv, nb * bs, D)[:, :sl].float()
        v = v_cache[blocks].permute(1, 0, 3, 2).reshape(Hkv, nb * bs, D)[:, :sl].float()
        if k_cache.dtype == torch.float8_e4m3fn:
            k, v = k * k_scale, v * v_scale
        k = k.repeat_interleave(G, dim=0)
        v = v.repeat_interleave(G, dim=0)
        qq = q[a:b].permute(1, 0, 2).float()                  # [Hq, ql, D]
        sc = torch.matmul(qq, k.transpose(1, 2)) * scale      # [Hq, ql, sl]
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        pos = torch.arange(sl - ql, sl, device=q.device)[:, None]
        key = torch.arange(sl, device=q.device)[None, :]
        if alibi is not None:
            sc = sc + alibi.float()[:, None, None] * (key - pos)[None].float()
        mask = (key <= pos) if causal else torch.ones((ql, sl), dtype=torch.bool, device=q.device)
        if window > 0:
            mask &= key > pos - window
        sc = sc.masked_fill(~mask[None], float("-inf"))
        if visible is not None:
            sc = sc.masked_fill(~visible(pos, key), float("-inf"))
        lse[:, a:b] = torch.logsumexp(sc, dim=-1)
        p = torch.softmax(sc, dim=-1)
        out[a:b] = torch.matmul(p, v).permute(1, 0, 2).to(q.dtype)
    return (out, lse) if return_lse else out


def sparse_step_selection(vert, vcount, slash, scount, key_base: int, q_base: int, ql: int, sl: int, causal: bool):
    """Which 32-key steps each 128-row query tile of one sequence visits, per head: bool [Hq, tiles, steps].
    A step is visited when it holds a selected key position, or when a selected diagonal (query position minus key
    position) crosses it inside the tile's rows; causal passes always visit the tile's own diagonal."""
    Hq = vert.shape[0]
    tiles, steps = (ql + 127) // 128, (sl + 31) // 32
    sel = torch.zeros((Hq, tiles, steps), dtype=torch.bool, device=vert.device)
    t = torch.arange(tiles, device=vert.device)
    qa0 = q_base + t * 128 - key_base                                        # [tiles] first / last row, on the key axis
    qa1 = q_base + torch.clamp((t + 1) * 128, max=ql) - 1 - key_base
    for h in range(Hq):
        k = vert[h, : int(vcount[h])].long() - key_base
        k = k[(k >= 0) & (k < sl)]
        sel[h, :, k // 32] = True
        d = slash[h, : int(scount[h])].long()
        d = d[d >= 0]
        bands = [(qa0[:, None] - d[None], qa1[:, None] - d[None])]
        if causal:
            bands.append((qa0[:, None], qa1[:, None]))
        for a, b in bands:
            a, b = a.clamp(min=0), b.clamp(max=sl - 1)
            for j in range(6):                                              # a band of <= 128 keys touches <= 5 steps
                st = a // 32 + j
                ok = (a <= b) & (st <= b // 32)
                ti = t[:, None].expand_as(st)[ok]
                sel[h, ti, st[ok]] = True
    return sel


def paged_attention_sparse(q, k_cache, v_cache, block_table, seq_lens, q_start_loc, scale, vert, vcount, slash, scount,
                           key_base, q_base, causal: bool = True, softcap: float = 0.0, k_scale: float = 1.0,
                           v_scale: float = 1.0):
    """Vertical-slash sparse attention at 32-key granularity (see ``sparse_step_selection``); vert / slash
    [S, Hq, N] with counts [S, Hq], key_base / q_base [S].  Returns (out [T, Hq, D], lse [Hq, T])."""
    out = torch.zeros_like(q)
    lse = torch.full((q.shape[1], q.shape[0]), float("-inf"), dtype=torch.float32, device=q.device)
    qsl, sls = q_start_loc.tolist(), seq_lens.tolist()
    for s, sl in enumerate(sls):
        a, b = qsl[s], qsl[s + 1]
        if a == b or sl == 0:
            continue
        sel = sparse_step_selection(vert[s], vcount[s], slash[s], scount[s], int(key_base[s]), int(q_base[s]), b - a, sl,
                                    causal)

        def visible(pos, key, sel=sel, lo=sl - (b - a)):
            return sel[:, (pos[:, 0] - lo) // 128][:, :, key[0] // 32]
        o, l = paged_attention(q[a:b], k_cache, v_cache, block_table[s:s + 1], seq_lens[s:s + 1],
                               torch.tensor([0, b - a], dtype=torch.int32, device=q.device), scale, softcap=softcap,
                               return_lse=True, k_scale=k_scale, v_scale=v_scale, causal=causal, visible=visible)
        out[a:b], lse[:, a:b] = torch.nan_to_num(o), l
    return out, lse


def merge_attn_states(prefix, prefix_lse, suffix, suffix_lse):
    """prefix/suffix: [T, H, D]; lse: [H, T]."""
    a = torch.where(torch.isposinf(prefix_lse), torch.full_like(prefix_lse, float("-inf")), prefix_lse)
    b = torch.where(torch.isposinf(suffix_lse), torch.full_like(suffix_lse, float("-inf")), suffix_lse)
    mx = torch.maximum(a, b)
    mu = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
    ea, eb = torch.exp(a - mu), torch.exp(b - mu)
    den = ea + eb
    wa = torch.where(den > 0, ea / den, torch.zeros_like(den)).T[..., None]
    wb = torch.where(den > 0, eb / den, torch.zeros_like(den)).T[..., None]
    out = (prefix.float() * wa + suffix.float() * wb).to(prefix.dtype)
    return out, torch.where(den > 0, mu + torch.log(den), torch.full_like(den, float("-inf")))


# ---- sampling ------------------------------------------------------------------
def apply_penalties(logits, prompt_mask, out_counts, rep, freq, pres):
    seen = prompt_mask.bool() | (out_counts > 0)
    r = rep[:, None]
    pen = torch.where(logits > 0, logits / r, logits * r)
    logits.copy_(torch.where(seen, pen, logits))
    logits.sub_(freq[:, None] * out_counts.float())
    logits.sub_(pres[:, None] * (out_counts > 0).float())
    return logits


def topk_topp_mask(logits, top_k=None, top_p=None, min_p=None):
    """In place -inf masking, sort based (the oracle for the radix kernel)."""
    S, V = logits.shape
    if top_k is not None:
        k = top_k.long().clone()
        k[(k <= 0) | (k > V)] = V
        srt = logits.sort(dim=-1, descending=True).values
        thr = srt.gather(1, (k - 1)[:, None])
        logits.masked_fill_(logits < thr, float("-inf"))
    if top_p is not None:
        probs = torch.softmax(logits, dim=-1)
        sp, si = probs.sort(dim=-1, descending=True)
        cum = sp.cumsum(-1)
        # smallest set whose mass reaches p; the first token is always kept
        drop = (cum - sp) >= top_p[:, None]
        drop[:, 0] = False
        thr = torch.where(drop, torch.full_like(sp, 2.0), sp).min(dim=-1, keepdim=True).values
        logits.masked_fill_(probs < thr, float("-inf"))
    if min_p is not None:
        probs = torch.softmax(logits, dim=-1)
        mx = probs.max(dim=-1, keepdim=True).values
        logits.masked_fill_(probs < min_p[:, None] * mx, float("-inf"))
    return logits


def sample(logits, temperature=None, top_k=None, top_p=None, min_p=None, seeds=None, generator=None):
    S, V = logits.shape
    out = logits.argmax(dim=-1)
    if temperature is None:
        return out
    rnd = temperature >= 1e-5
    if not bool(rnd.any()):
        return out
    z = logits.float() / torch.where(rnd, temperature, torch.ones_like(temperature))[:, None]
    z = topk_topp_mask(z, top_k, top_p, min_p)
    probs = torch.softmax(z, dim=-1)
    if seeds is not None:
        draws = torch.empty(S, dtype=torch.long, device=logits.device)
        for i in range(S):
            g = torch.Generator(device=logits.device)
            g.manual_seed(int(seeds[i]) & 0x7FFFFFFFFFFFFFFF)
            draws[i] = torch.multinomial(probs[i], 1, generator=g)[0]
    else:
        draws = torch.multinomial(probs, 1, generator=generator)[:, 0]
    return torch.where(rnd, draws, out)


# ---- fp8 -------------------------------------------------------------------------
def scaled_fp8_quant(x, scale=None):
    if scale is None:
        scale = (x.abs().max().float() / FP8_MAX).clamp(min=1e-12).reshape(1)
    q = (x.float() / scale).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scale


def per_token_fp8_quant(x, scale_ub=None):
    amax = x.abs().amax(dim=-1, keepdim=True).float()
    if scale_ub is not None:
        amax = amax.clamp(max=float(scale_ub))
    scale = (amax / FP8_MAX).clamp(min=1.0 / (FP8_MAX * 512.0))
    q = (x.float() / scale).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scale


def fp8_dequant(q, scale, dtype):
    return (q.float() * scale).to(dtype)


def per_group_fp8_quant(x, group: int = 128):
    """One dynamic scale per ``group`` consecutive elements of a row (the last group may be short)."""
    K = x.shape[-1]
    ng = -(-K // group)
    xf = x.float()
    pad = ng * group - K
    if pad:
        xf = F.pad(xf, (0, pad))
    g = xf.reshape(*x.shape[:-1], ng, group)
    scale = (g.abs().amax(dim=-1, keepdim=True) / FP8_MAX).clamp(min=1.0 / (FP8_MAX * 512.0))
    q = (g / scale).clamp(-FP8_MAX, FP8_MAX).reshape(*x.shape[:-1], ng * group)[..., :K].to(torch.float8_e4m3fn)
    return q, scale.squeeze(-1)


def expand_block_scales(scale: torch.Tensor, rows: int, cols: int, block: int = 128) -> torch.Tensor:
    """[.., ceil(rows/block), ceil(cols/block)] block scales -> one scale per element [.., rows, cols]."""
    s = scale.repeat_interleave(block, dim=-2).repeat_interleave(block, dim=-1)
    return s[..., :rows, :cols]


def fp8_gemm(xq, w, x_scale, w_scale, out_dtype, bias=None, block: bool = False):
    M, K = xq.shape
    if block:
        xf = xq.float() * x_scale.reshape(M, -1).float().repeat_interleave(128, dim=1)[:, :K]
        wf = w.float() * expand_block_scales(w_scale.float(), w.shape[0], K)
    else:
        xf = xq.float() * (x_scale.reshape(-1, 1).float() if x_scale.numel() == M else x_scale.reshape(()).float())
        wf = w.float() * w_scale.reshape(()).float()
    y = xf @ wf.t()
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype)


def skinny_gemm(x, w, bias=None, w_scale=None):
    if w.dtype == torch.float8_e4m3fn:
        w = (w.float() * (w_scale.float() if w_scale is not None else 1.0)).to(x.dtype)
    return F.linear(x, w, bias)


# ---- mixture of experts ------------------------------------------------------------------
def moe_topk_softmax(logits: torch.Tensor, k: int, renormalize: bool):
    probs = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(probs, k, dim=-1)
    if renormalize:
        w = w / w.sum(dim=-1, keepdim=True)
    return w, ids.to(torch.int32)


def fused_moe(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, topk_w: torch.Tensor, topk_ids: torch.Tensor,
              w13_scale: Optional[torch.Tensor] = None, w2_scale: Optional[torch.Tensor] = None,
              block_scales: bool = False, activation: str = "silu", act_limit: float = 0.0,
              gated: bool = True) -> torch.Tensor:
    """out[t] = sum_j topk_w[t, j] * W2_e( act(Wg_e x_t) * (Wu_e x_t) ), e = topk_ids[t, j];
    negative ids (expert on another rank) contribute nothing.  fp32 accumulation.  ``block_scales``:
    the weight scales are per 128 x 128 block instead of per expert.  ``gated=False``: experts without a gate half,
    W2_e act(Wu_e x_t), w13 [E, I, H]."""
    T, H = x.shape
    E, I2, _ = w13.shape
    I = I2 // 2 if gated else I2
    out = torch.zeros((T, w2.shape[1]), dtype=torch.float32, device=x.device)
    xf = x.float()
    for e in range(E):
        tok, slot = torch.where(topk_ids == e)
        if tok.numel() == 0:
            continue
        if block_scales:
            a = w13[e].float() * expand_block_scales(w13_scale[e].float(), I2, H)
            b = w2[e].float() * expand_block_scales(w2_scale[e].float(), w2.shape[1], I)
        else:
            a = w13[e].float() * (w13_scale[e].float() if w13_scale is not None else 1.0)
            b = w2[e].float() * (w2_scale[e].float() if w2_scale is not None else 1.0)
        xe = xf[tok]
        if block_scales:      # what the device kernels do: activations rounded to e4m3 per group of 128
            q, s_ = per_group_fp8_quant(xe.to(x.dtype))
            xe = (q.float().view(*s_.shape, -1) * s_.unsqueeze(-1)).view(xe.shape)
        h = xe @ a.t()
        if not gated:
            act = _act(activation, h).to(x.dtype).float()
        elif activation == "clamped_swiglu":
            act = clamped_swiglu(h[:, :I], h[:, I:], act_limit).to(x.dtype).float()
        else:
            act = (_act(activation, h[:, :I]) * h[:, I:]).to(x.dtype).float()
        if block_scales:
            q, s_ = per_group_fp8_quant(act.to(x.dtype))
            act = (q.float().view(*s_.shape, -1) * s_.unsqueeze(-1)).view(act.shape)
        out.index_add_(0, tok, (act @ b.t()) * topk_w[tok, slot].float().unsqueeze(1))
    return out.to(x.dtype)


def int8_quant(x, scale=None):
    xf = x.float()
    if scale is None:
        s = (xf.abs().amax(-1, keepdim=True) / 127.0).clamp(min=1e-10)
    else:
        s = scale.float().reshape(())
    q = torch.round(xf / s).clamp(-128, 127).to(torch.int8)
    return q, (s if scale is None else scale)


def int8_quant_azp(x, scale=None, azp=None):
    xf = x.float()
    if scale is None:
        mx, mn = xf.amax(-1, keepdim=True), xf.amin(-1, keepdim=True)
        s = ((mx - mn) / 255.0).clamp(min=1e-10)
        z = torch.round(-128.0 - mn / s).to(torch.int32)
        q = (torch.round(xf / s) + z).clamp(-128, 127).to(torch.int8)
        return q, s, z
    s = scale.float().reshape(())
    z = azp.reshape(()).to(torch.int32) if azp is not None else torch.zeros((), dtype=torch.int32, device=x.device)
    q = (torch.round(xf / s) + z).clamp(-128, 127).to(torch.int8)
    return q, scale, azp


# ---- state-space layers ---------------------------------------------------------------------------
def causal_conv1d(x, weight, bias, conv_state, qsl, seq_lens, block_table, activation=True):
    T, C = x.shape
    W = weight.shape[1]
    out = torch.zeros((T, C), dtype=x.dtype, device=x.device)
    w = weight.float()
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        if sl <= 0:
            continue
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        L = t1 - t0
        slot = int(block_table[s, 0])
        prev = conv_state[slot].float() if sl - L > 0 else torch.zeros((C, W - 1), device=x.device)
        seq = torch.cat([prev.t(), x[t0:t1].float()], dim=0)              # [W-1+L, C]
        win = seq.unfold(0, W, 1)                                           # [L, C, W]
        y = (win * w.unsqueeze(0)).sum(-1)
        if bias is not None:
            y = y + bias.float()
        if activation:
            y = torch.nn.functional.silu(y)
        out[t0:t1] = y.to(x.dtype)
        conv_state[slot] = seq[-(W - 1):].t().to(conv_state.dtype)
    return out


def selective_scan(u, delta, A, B, C, D, z, delta_bias, ssm_state, qsl, seq_lens, block_table, softplus=True,
                   num_groups=1):
    T, Ch = u.shape
    Nst = ssm_state.shape[2]
    E = delta.shape[1]
    rep = Ch // E
    out = torch.zeros((T, Ch), dtype=u.dtype, device=u.device)
    A_full = (A.float().repeat_interleave(rep).unsqueeze(1).expand(Ch, Nst) if A.dim() == 1 else A.float())
    Dv = D.float().repeat_interleave(rep) if D is not None else None
    gch = Ch // num_groups
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        if sl <= 0:
            continue
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        slot = int(block_table[s, 0])
        h = ssm_state[slot].float().clone() if sl - (t1 - t0) > 0 else torch.zeros((Ch, Nst), device=u.device)
        for t in range(t0, t1):
            dt = delta[t].float()
            if delta_bias is not None:
                dt = dt + delta_bias.float()
            if softplus:
                dt = torch.nn.functional.softplus(dt)
            dt = dt.repeat_interleave(rep)                                   # [Ch]
            x = u[t].float()
            Bt = B[t].float().view(num_groups, Nst).repeat_interleave(gch, dim=0)   # [Ch, N]
            Ct = C[t].float().view(num_groups, Nst).repeat_interleave(gch, dim=0)
            h = torch.exp(dt.unsqueeze(1) * A_full) * h + (dt * x).unsqueeze(1) * Bt
            y = (h * Ct).sum(-1)
            if Dv is not None:
                y = y + Dv * x
            if z is not None:
                y = y * torch.nn.functional.silu(z[t].float())
            out[t] = y.to(u.dtype)
        ssm_state[slot] = h
    return out


# ---- 4-bit weights -----------------------------------------------------------------------------------
def w4_unpack(qw: torch.Tensor) -> torch.Tensor:
    """int32 [N, K/8] in the kernel's nibble order -> int64 [N, K] of values 0..15."""
    w = qw.to(torch.int64) & 0xFFFFFFFF
    cols = [(w >> (4 * (e // 2 + 4 * (e % 2)))) & 0xF for e in range(8)]
    return torch.stack(cols, dim=-1).reshape(qw.shape[0], -1)


def cb4_dequant(codes, scales, table, group, hi_first, dtype):
    N_, K2 = codes.shape
    first, second = (codes >> 4, codes & 15) if hi_first else (codes & 15, codes >> 4)
    idx = torch.stack((first, second), dim=-1).reshape(N_, 2 * K2).long()
    vals = table.float()[idx].view(N_, -1, group) * scales.float().unsqueeze(-1)
    return vals.view(N_, 2 * K2).to(dtype)


def w4_dequant(qw, scales, zeros, group, dtype):
    q = w4_unpack(qw).float()
    s = scales.float().repeat_interleave(group, dim=1)
    z = zeros.float().repeat_interleave(group, dim=1)
    return ((q - z) * s).to(dtype)


# ---- multi-LoRA --------------------------------------------------------------------------------------
def lora_update(y, x, A, B, tok_slot):
    for s in torch.unique(tok_slot).tolist():
        if s < 0:
            continue
        idx = torch.nonzero(tok_slot == s).squeeze(1)
        d = (x[idx].float() @ A[s].float().t()) @ B[s].float().t()
        y[idx] = (y[idx].float() + d).to(y.dtype)


# ---- multi-head latent attention -----------------------------------------------------------------------
def mla_cache_write(kv_c, k_pe, kc, vt, slot_mapping, kv_scale=1.0):
    BS = kc.shape[1]
    Rk = kv_c.shape[1]
    if kc.dtype == torch.float8_e4m3fn:
        kv_c, k_pe = kv_c.float() / kv_scale, k_pe.float() / kv_scale
    for t in range(kv_c.shape[0]):
        slot = int(slot_mapping[t])
        if slot < 0:
            continue
        b, o = slot // BS, slot % BS
        kc[b, o, :Rk] = kv_c[t].to(kc.dtype)
        kc[b, o, Rk:] = k_pe[t].to(kc.dtype)
        vt[b, :, o] = kv_c[t].to(vt.dtype)


def mla_attention(q, kc, vt, block_table, seq_lens, q_start_loc, scale, kv_scale=1.0, window=0, sink=None):
    """``sink`` fp32 [H]: exp(sink[h]) joins head h's softmax denominator (no key, no value)."""
    T, H, DK = q.shape
    DV, BS = vt.shape[1], kc.shape[1]
    if kc.dtype != torch.float8_e4m3fn:
        kv_scale = 1.0
    out = torch.zeros((T, H, DV), dtype=q.dtype, device=q.device)
    for s in range(seq_lens.shape[0]):
        L = int(seq_lens[s])
        a, b = int(q_start_loc[s]), int(q_start_loc[s + 1])
        if L <= 0 or b <= a:
            continue
        nblk = (L + BS - 1) // BS
        blocks = block_table[s, :nblk].long()
        K = kc[blocks].reshape(-1, DK)[:L].float() * kv_scale              # [L, DK]
        V = vt[blocks].permute(0, 2, 1).reshape(-1, DV)[:L].float() * kv_scale   # [L, DV]
        qs = q[a:b].float()                                                # [n, H, DK]
        n = b - a
        sc = torch.einsum("nhd,ld->nhl", qs, K) * scale
        pos = torch.arange(L, device=q.device).view(1, 1, L)
        lim = (L - n + torch.arange(n, device=q.device) + 1).view(n, 1, 1)
        sc = sc.masked_fill(pos >= lim, float("-inf"))
        if window > 0:
            sc = sc.masked_fill(pos < lim - window, float("-inf"))
        out[a:b] = torch.einsum("nhl,ld->nhd", softmax_with_sink(sc, sink.view(1, H, 1) if sink is not None else None),
                                V).to(q.dtype)
    return out


def softmax_with_sink(sc, sink=None):
    """Softmax over the last dimension; ``sink`` (broadcastable to sc[..., :1]) adds exp(sink) to the denominator."""
    if sink is None:
        return torch.softmax(sc, dim=-1)
    mx = torch.maximum(sc.max(-1, keepdim=True).values, sink.float())
    e = torch.exp(sc - mx)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink.float() - mx))


# ---- residual streams (hyper-connections) ---------------------------------------------------------
def stream_embed(ids, weight, scale: float, streams: int):
    """fp32 residual streams [streams, T, W], every one a copy of ``weight[ids] * scale``."""
    x = weight[ids.long()].float() * scale
    return x.unsqueeze(0).repeat(streams, 1, 1)


def stream_mix_norm(xs, w_in, gain, eps: float, out_dtype):
    """h = u / sqrt(mean(u^2) + eps) * gain with u = sum_s w_in[s] xs[s]; one gain for the whole row."""
    u = (xs.float() * w_in.float().view(-1, 1, 1)).sum(0)
    h = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * gain.float()
    return h.to(out_dtype)


def stream_update(xs, y, mix, w_out):
    """xs[t] <- sum_s mix[s, t] xs[s] + w_out[t] * y for all t at once, in place."""
    new = torch.einsum("st,snw->tnw", mix.float(), xs.float()) + w_out.float().view(-1, 1, 1) * y.float().unsqueeze(0)
    xs.copy_(new)
    return xs


# ---- sigmoid attention with mixed head scores over a window plus kept first tokens ------------------
def unit_rms_qk_and_cache(qkv, H: int, G: int, D: int, Dv: int, eps: float, k_cache, v_cache, slot_mapping):
    """qkv [T, H*D + G*D + G*Dv] -> q / rms(q) per head as [T, H, D] (qkv's type); k / rms(k) and v go to the cache
    (k_cache [blocks, G, bs, D], v_cache [blocks, G, Dv, bs]) at ``slot_mapping`` (negative: not stored)."""
    T = qkv.shape[0]
    q = qkv[:, : H * D].float().view(T, H, D)
    k = qkv[:, H * D: (H + G) * D].float().view(T, G, D)
    v = qkv[:, (H + G) * D:].view(T, G, Dv)
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
    if k_cache is not None:
        bs = k_cache.shape[2]
        ok = slot_mapping[:T] >= 0
        sl = slot_mapping[:T][ok].long()
        k_cache[sl // bs, :, sl % bs] = k[ok].to(k_cache.dtype)
        v_cache[sl // bs, :, :, sl % bs] = v[ok].to(v_cache.dtype)
    return q.to(qkv.dtype)


def sigmoid_window_attention(qn, k_cache, v_cache, block_table, seq_lens, qsl, talk, pb, scale: float, window: int,
                             keep_first: int, out_dtype):
    """Per sequence: raw[g, i, j] = scale * qn[i, g] . k[j, kv(g)]; mixed[h] = sum_g talk[h, g] raw[g];
    weight = sigmoid(mixed + pb[h]) on the visible keys (j <= i and (i - j < window or j < keep_first); window 0 =
    every earlier key), no normalisation over keys; out[i, h] = sum_j weight[h, i, j] v[j, kv(h)]."""
    T, H, D = qn.shape
    G, Dv, bs = v_cache.shape[1], v_cache.shape[2], v_cache.shape[3]
    out = torch.zeros((T, H, Dv), dtype=torch.float32, device=qn.device)
    rep = H // G
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        L = t1 - t0
        if sl <= 0 or L <= 0:
            continue
        nb = -(-sl // bs)
        blocks = block_table[s, :nb].long()
        k = k_cache[blocks].float().permute(0, 2, 1, 3).reshape(nb * bs, G, D)[:sl]
        v = v_cache[blocks].float().permute(0, 3, 1, 2).reshape(nb * bs, G, Dv)[:sl]
        kk, vv = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
        raw = torch.einsum("ihd,jhd->hij", qn[t0:t1].float(), kk) * scale
        mixed = torch.einsum("hg,gij->hij", talk.float(), raw)
        i = torch.arange(sl - L, sl, device=qn.device)[:, None]
        j = torch.arange(sl, device=qn.device)[None, :]
        vis = j <= i
        if window > 0:
            vis = vis & ((i - j < window) | (j < keep_first))
        w = torch.sigmoid(mixed + pb.float().view(-1, 1, 1)) * vis
        out[t0:t1] = torch.einsum("hij,jhd->ihd", w, vv)
    return out.view(T, H * Dv).to(out_dtype)


# ---- gated delta rule with one decay per key channel ---------------------------------------------------
def gated_delta_rule(qkv, a_raw, b_raw, gate_raw, a_log, dt_bias, norm_w, state, qsl, seq_lens, slot_table,
                     H: int, G: int, D: int, Dv: int, eps: float):
    """qkv [T, 2*G*D + H*Dv] (after the short convolution), a_raw [T, H*D], b_raw [T, H], gate_raw [T, H*Dv];
    state fp32 [slots, H, Dv, D] (S transposed), updated in place.  Per token and head (q, k of head h // (H / G)):
    q <- q / sqrt(|q|^2 + 1e-6) / sqrt(D), k <- k / sqrt(|k|^2 + 1e-6), decay = exp(-exp(a_log[h]) *
    softplus(a_raw + dt_bias)); S <- decay[:, None] * S; u = sigmoid(b) * (v - S^T k); S <- S + k u^T; o = S^T q;
    out = o / rms(o) * norm_w * sigmoid(gate_raw)."""
    T = qkv.shape[0]
    out = torch.zeros((T, H, Dv), dtype=torch.float32, device=qkv.device)
    rep = H // G
    q = qkv[:, : G * D].float().view(T, G, D)
    k = qkv[:, G * D: 2 * G * D].float().view(T, G, D)
    v = qkv[:, 2 * G * D:].float().view(T, H, Dv)
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(b_raw.float())
    decay = torch.exp(-torch.exp(a_log.float()).view(1, H, 1)
                      * torch.nn.functional.softplus(a_raw.float() + dt_bias.float()).view(T, H, D))
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        if sl <= 0 or t1 <= t0:
            continue
        slot = int(slot_table[s, 0])
        S = state[slot].transpose(1, 2).clone() if sl - (t1 - t0) > 0 else \
            torch.zeros((H, D, Dv), dtype=torch.float32, device=qkv.device)
        for t in range(t0, t1):
            S = decay[t].unsqueeze(-1) * S
            u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
            S = S + k[t].unsqueeze(-1) * u.unsqueeze(1)
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S.transpose(1, 2)
    o = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    o = o * torch.sigmoid(gate_raw.float().view(T, H, Dv))
    return o.view(T, H * Dv).to(qkv.dtype)


# ---- fp32 residual with a norm after and before every sub-layer ---------------------------------------------
def residual_norms(x, y, w_post, w_pre, eps: float, out_dtype, gain_offset: float = 1.0):
    """x fp32 [T, W], in place: x += y / rms(y) * (gain_offset + w_post) when ``y`` is given; returns
    x / rms(x) * (gain_offset + w_pre) in ``out_dtype`` when ``w_pre`` is given."""
    if y is not None:
        f = y.float()
        x += f * torch.rsqrt(f.pow(2).mean(-1, keepdim=True) + eps) * (gain_offset + w_post.float())
    if w_pre is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (gain_offset + w_pre.float())).to(out_dtype)


def gated_residual_group_norm(x, subs, w_next, groups: int, eps: float, out_dtype):
    """x fp32 [T, W], in place: x += sum over ``subs`` of y * scale * sigmoid(gate), one tuple (y, scale, gate, extra,
    extra_w) per sub-layer (scale fp32 [W] or None, gate [T, W] pre-activations or None, extra [T, W] with extra_w fp32
    [T] or None: y + extra_w[:, None] * extra takes y's place); the sub-layers' terms are summed before they join x.
    With ``w_next`` returns every one of ``groups`` equal parts of the updated row divided by its own root mean square,
    times w_next, in ``out_dtype``."""
    total = None
    for y, scale, gate, extra, extra_w in subs:
        f = y.float()
        if extra is not None:
            f = f + extra_w.float().view(-1, 1) * extra.float()
        if scale is not None:
            f = f * scale.float()
        if gate is not None:
            f = f * torch.sigmoid(gate.float())
        total = f if total is None else total + f
    if total is not None:
        x += total
    if w_next is None:
        return None
    T, W = x.shape
    p = x.view(T, groups, W // groups)
    return ((p * torch.rsqrt(p.pow(2).mean(-1, keepdim=True) + eps)).view(T, W) * w_next.float()).to(out_dtype)


# ---- latent attention over a window: cache write and attention ----------------------------------------------
def rotate_interleaved(x, cos, sin):
    """x [..., 2n] as pairs (x[2i], x[2i+1]) turned by the angles whose cos / sin [..., n] are given (fp32)."""
    u, v = x[..., 0::2].float(), x[..., 1::2].float()
    return torch.stack((u * cos - v * sin, v * cos + u * sin), dim=-1).flatten(-2)


def latent_norm_rope_cache(q, down, c_weight, cos_sin, positions, qf, kc, slot_mapping, H: int, D: int, P: int,
                           R: int, rot_dims: int, eps: float, vt=None):
    """q [T, H * (D + P)], down [T, R + P]; cos_sin fp32 [positions, rot_dims] (cosines then sines).
    Cache row of a token = [rms(down[:R]) * c_weight | rotated down[R:]] -> kc [blocks, bs, R + P] at slot_mapping;
    the rotated last P values of every query head go to qf[:, h, R:] (qf [T, H, R + P])."""
    T = q.shape[0]
    cs = cos_sin[positions[:T].long()]
    half = rot_dims // 2
    cos, sin = cs[:, :half], cs[:, half:]
    c = down[:, :R].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * c_weight.float()
    kr = down[:, R:].float().clone()
    kr[:, :rot_dims] = rotate_interleaved(kr[:, :rot_dims], cos, sin)
    qr = q.view(T, H, D + P)[:, :, D:].float().clone()
    qr[:, :, :rot_dims] = rotate_interleaved(qr[:, :, :rot_dims], cos[:, None], sin[:, None])
    qf[:, :, R:] = qr.to(qf.dtype)
    if kc is not None:
        bs = kc.shape[1]
        ok = slot_mapping[:T] >= 0
        sl = slot_mapping[:T][ok].long()
        kc[sl // bs, sl % bs] = torch.cat([c, kr], -1)[ok].to(kc.dtype)
        if vt is not None and vt.numel():
            vt[sl // bs, :, sl % bs] = c[ok].to(vt.dtype)


def latent_window_attention(q, kc, block_table, seq_lens, qsl, scale: float, window: int, R: int, sink=None):
    """q [T, H, DK] against the latent rows kc [blocks, bs, DK]: softmax over the keys j <= i with i - j < window
    (window 0: all of them) of scale * q . row; returns the weighted sums of the rows' first R values, [T, H, R].
    ``sink`` fp32 [H]: exp(sink[h]) joins head h's denominator (no key, no value)."""
    T, H, DK = q.shape
    bs = kc.shape[1]
    out = torch.zeros((T, H, R), dtype=torch.float32, device=q.device)
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        L = t1 - t0
        if sl <= 0 or L <= 0:
            continue
        nb = -(-sl // bs)
        rows = kc[block_table[s, :nb].long()].reshape(nb * bs, DK)[:sl].float()
        sc = torch.einsum("ihd,jd->hij", q[t0:t1].float(), rows) * scale
        i = torch.arange(sl - L, sl, device=q.device)[:, None]
        j = torch.arange(sl, device=q.device)[None, :]
        vis = j <= i
        if window > 0:
            vis = vis & (i - j < window)
        sc = sc.masked_fill(~vis[None], float("-inf"))
        out[t0:t1] = torch.einsum("hij,jd->ihd", softmax_with_sink(sc, sink.view(H, 1, 1) if sink is not None else None),
                                  rows[:, :R])
    return out.to(q.dtype)


# ---- matrix memory with exponential gates and a running maximum (mLSTM) --------------------------------------
def mlstm(proj, i_bias, f_bias, norm_w, state_nm, state_s, qsl, seq_lens, slot_table, H: int, D: int, Dv: int,
          cap: float, eps: float):
    """proj [T, 2*H*D + 2*H*Dv + 2*H] = [q | k | v | output gate | input gate | forget gate] (pre-activations);
    state_nm fp32 [slots, H, Dn] (n in [:D], the running maximum at [D]); state_s fp32 [slots, H, D, Dv].
        i = cap tanh((i_raw + i_bias) / cap), f = logsigmoid(cap tanh((f_raw + f_bias) / cap))
        m' = max(f + m, i); S' = e^(f + m - m') S + e^(i - m') k v^T; n' likewise with k
        o = S'^T q D^-1/2 / (max(|n' . q D^-1/2|, e^-m') + 1e-6)
    out = o / rms(o) per head * norm_w * sigmoid(output gate)."""
    T = proj.shape[0]
    HD, HV = H * D, H * Dv
    q = proj[:, :HD].float().view(T, H, D) * D ** -0.5
    k = proj[:, HD: 2 * HD].float().view(T, H, D)
    v = proj[:, 2 * HD: 2 * HD + HV].float().view(T, H, Dv)
    og = proj[:, 2 * HD + HV: 2 * HD + 2 * HV].float()
    ig = cap * torch.tanh((proj[:, 2 * HD + 2 * HV: 2 * HD + 2 * HV + H].float() + i_bias.float()) / cap)
    fg = F.logsigmoid(cap * torch.tanh((proj[:, 2 * HD + 2 * HV + H:].float() + f_bias.float()) / cap))
    out = torch.zeros((T, H, Dv), dtype=torch.float32, device=proj.device)
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        if sl <= 0 or t1 <= t0:
            continue
        slot = int(slot_table[s, 0])
        if sl - (t1 - t0) > 0:
            S, n, m = state_s[slot].clone(), state_nm[slot, :, :D].clone(), state_nm[slot, :, D].clone()
        else:
            S = torch.zeros((H, D, Dv), dtype=torch.float32, device=proj.device)
            n, m = S.new_zeros((H, D)), S.new_zeros((H,))
        for t in range(t0, t1):
            m2 = torch.maximum(fg[t] + m, ig[t])
            a, b = torch.exp(fg[t] + m - m2), torch.exp(ig[t] - m2)
            S = a[:, None, None] * S + b[:, None, None] * k[t].unsqueeze(-1) * v[t].unsqueeze(1)
            n = a[:, None] * n + b[:, None] * k[t]
            m = m2
            den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
        state_s[slot] = S
        state_nm[slot, :, :D] = n
        state_nm[slot, :, D] = m
    o = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps)
    o = o.view(T, HV) * norm_w.float() * torch.sigmoid(og)
    return o.to(proj.dtype)


# ---- fp32 residual with a layer norm on every sub-layer's output -------------------------------------------------
def residual_layer_norm(x, y, weight, bias, eps: float, out_dtype, y2=None, y2_gate=None):
    """x fp32 [T, W].  With ``y`` (a sub-layer's output): x += (y - mean) / sqrt(var + eps) * weight + bias, in place, and
    x comes back in ``out_dtype`` (the next sub-layer reads the residual itself).  Without: the layer norm of x comes
    back in ``out_dtype`` and x stays.  ``y2`` / ``y2_gate`` [T, 1]: the sub-layer's output is y + y2 * sigmoid(gate)."""
    src = y.float() if y is not None else x
    if y2 is not None:
        src = src + y2.float() * torch.sigmoid(y2_gate.float().reshape(-1, 1))
    mu = src.mean(-1, keepdim=True)
    d = src - mu
    n = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    if bias is not None:
        n = n + bias.float()
    if y is None:
        return n.to(out_dtype)
    x += n
    return x if out_dtype == torch.float32 else x.to(out_dtype)


# ---- softmax attention with per-head q / k norms, part-rotated heads, several score maps and a choice of masks ---
def rotate_halves(x, cos, sin, rot: int):
    """x [..., D]: value i < rot / 2 is paired with value i + rot / 2 and the pair turned by the angle whose cos / sin
    [..., rot / 2] are given (fp32); values from ``rot`` on pass unchanged."""
    half = rot // 2
    u, v = x[..., :half].float(), x[..., half:rot].float()
    return torch.cat((u * cos - v * sin, v * cos + u * sin, x[..., rot:].float()), dim=-1)


def position_temperature(positions, coef: float, every: int):
    """fp32 [T]: 1 + coef * ln(floor((p + 1) / every) + 1), the factor queries at position p are multiplied by."""
    return 1.0 + float(coef) * torch.log((torch.div(positions.long() + 1, int(every), rounding_mode="floor") + 1).float())


def qk_norm_rope_cache(qkv, H: int, G: int, D: int, Dv: int, maps: int, q_weight, k_weight, cos_sin, positions,
                       rot: int, eps: float, k_cache, v_cache, slot_mapping, pairing: str = "halves", q_temp=None,
                       v_first=None, v_lam=None):
    """qkv [T, H*maps*D + G*maps*D + G*Dv].  Every D-wide map of every query / key head is divided by its root mean
    square, multiplied by q_weight / k_weight [D] and its first ``rot`` values are rotated (cos_sin fp32 [positions, rot],
    cosines then sines; ``pairing``: value i with i + rot / 2, "halves", or 2i with 2i + 1, "neighbours").  ``q_temp`` =
    (coef, every): queries times ``position_temperature``.  ``v_first`` [T, G * Dv] with ``v_lam`` (one fp32 value):
    the values become (1 - lam) v + lam v_first before they are cached.  Returns q [T, H, maps * D]; keys go to
    k_cache [blocks, G, bs, maps * D] and values to v_cache [blocks, G, Dv, bs] at ``slot_mapping``."""
    T = qkv.shape[0]
    nq, nk = H * maps * D, G * maps * D
    q = qkv[:, :nq].float().view(T, H * maps, D)
    k = qkv[:, nq: nq + nk].float().view(T, G * maps, D)
    v = qkv[:, nq + nk:].view(T, G, Dv)
    if v_first is not None:
        lam = v_lam.float().reshape(())
        v = ((1.0 - lam) * v.float() + lam * v_first[:T].float().view(T, G, Dv))
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_weight.float()
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_weight.float()
    if rot > 0:
        cs = cos_sin[positions[:T].long()]
        cos, sin = cs[:, None, : rot // 2], cs[:, None, rot // 2: rot]
        if pairing == "neighbours":
            q = torch.cat((rotate_interleaved(q[..., :rot], cos, sin), q[..., rot:]), -1)
            k = torch.cat((rotate_interleaved(k[..., :rot], cos, sin), k[..., rot:]), -1)
        else:
            q, k = rotate_halves(q, cos, sin, rot), rotate_halves(k, cos, sin, rot)
    if q_temp is not None:
        q = q * position_temperature(positions[:T], q_temp[0], q_temp[1]).view(T, 1, 1)
    qn = q.to(qkv.dtype).view(T, H, maps * D)
    if k_cache is not None:
        bs = k_cache.shape[2]
        ok = slot_mapping[:T] >= 0
        slots = slot_mapping[:T][ok].long()
        k_cache[slots // bs, :, slots % bs] = k.to(k_cache.dtype).view(T, G, maps * D)[ok]
        v_cache[slots // bs, :, :, slots % bs] = v.to(v_cache.dtype)[ok]
    return qn


def masked_softmax_attention(qn, k_cache, v_cache, block_table, seq_lens, qsl, scale: float, window: int, chunk: int,
                             sink, maps: int, lam, eps: float, out_scale: float, gate, out_dtype, softcap: float = 0.0,
                             dist_bias=None):
    """Softmax attention of qn [T, H, maps * D] over the paged keys (k_cache [blocks, G, bs, maps * D], v_cache [blocks,
    G, Dv, bs]); head h reads key / value head h // (H / G).  Key j is visible to the query at position i when j <= i,
    i - j < window (window > 0) and j // chunk == i // chunk (chunk > 0).  ``sink`` fp32 [H]: exp(sink[h]) joins the
    softmax denominator of head h (no key, no value).  maps == 2: each half of a head's row is an attention map of
    its own over the same values, combined as o = a1 - lam * a2 (lam: fp32 tensor of one element), divided by its
    root mean square over Dv and multiplied by out_scale.  ``gate`` [T, H * Dv]: the result is multiplied by its
    sigmoid.  ``softcap`` > 0: score <- softcap * tanh(score / softcap).  ``dist_bias`` fp32 [far + 1, H]: row
    min(i - j, far) is added to the (capped) scores of every head.  Returns [T, H * Dv] in ``out_dtype``."""
    T, H, MD = qn.shape
    D = MD // maps
    G, Dv, bs = v_cache.shape[1], v_cache.shape[2], v_cache.shape[3]
    rep = H // G
    out = torch.zeros((T, H, Dv), dtype=torch.float32, device=qn.device)
    for s in range(seq_lens.shape[0]):
        sl = int(seq_lens[s])
        t0, t1 = int(qsl[s]), int(qsl[s + 1])
        L = t1 - t0
        if sl <= 0 or L <= 0:
            continue
        nb = -(-sl // bs)
        blocks = block_table[s, :nb].long()
        keys = k_cache[blocks].permute(1, 0, 2, 3).reshape(G, nb * bs, MD)[:, :sl].float()
        vals = v_cache[blocks].permute(1, 0, 3, 2).reshape(G, nb * bs, Dv)[:, :sl].float()
        i = torch.arange(sl - L, sl, device=qn.device)[:, None]
        j = torch.arange(sl, device=qn.device)[None, :]
        vis = j <= i
        if window > 0:
            vis = vis & (i - j < window)
        if chunk > 0:
            vis = vis & (i // chunk == j // chunk)
        q = qn[t0:t1].float().view(L, G, rep, maps, D)
        sc = torch.einsum("igrmd,gjmd->grmij", q, keys.view(G, sl, maps, D)) * scale
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        if dist_bias is not None:
            far = dist_bias.shape[0] - 1
            b = dist_bias.float()[(i - j).clamp(0, far)]                    # [L, sl, H]
            sc = sc + b.permute(2, 0, 1).reshape(G, rep, 1, L, sl)
        sc = sc.masked_fill(~vis, float("-inf"))
        mx = sc.max(-1, keepdim=True).values
        if sink is not None:
            sk = sink.float().view(G, rep, 1, 1, 1)
            mx = torch.maximum(mx, sk)
        e = torch.exp(sc - mx)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sk - mx)
        a = torch.einsum("grmij,gjd->igrmd", e / den, vals)                  # [L, G, rep, maps, Dv]
        if maps == 2:
            o = a[..., 0, :] - lam.float().reshape(()) * a[..., 1, :]
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * out_scale
        else:
            o = a[..., 0, :]
        out[t0:t1] = o.reshape(L, H, Dv)
    out = out.view(T, H * Dv)
    if gate is not None:
        out = out * torch.sigmoid(gate[:T].float())
    return out.to(out_dtype)


def fp32_rows_dot(x, weight, bias):
    """x [T, W] (any type) against fp32 rows weight [R, W] (+ bias [R]) in fp32: [T, R]."""
    out = x.float() @ weight.float().t()
    return out + bias.float() if bias is not None else out
