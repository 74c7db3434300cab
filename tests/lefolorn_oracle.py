"""A slow, whole-sequence implementation of the Lefolorn design, one function per mechanism, written from its equations
and sharing no code with the package: the oracle of tests/test_lefolorn.py.  Everything runs in fp32 (or fp64) on the
CPU over one whole sequence at a time; there is no cache, no batching and no portioning here.

Notation: x residual [L, W]; a layer computes h = N(x), x <- x + a1 * r1(h) * mixer(h) + a2 * r2(h) * ff(h) with
N a norm in groups, a1 / a2 per-channel scales and r(h) = sigmoid(R h + b) per-channel gates.
"""
import json
import math
import os

import torch


# ---- norms ---------------------------------------------------------------------------------------------------------
def unit_rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """Every one of ``groups`` equal consecutive parts of a row divided by its own RMS; one weight over the row."""
    L, W = x.shape
    return unit_rms(x.reshape(L, groups, W // groups), eps).reshape(L, W) * w


# ---- positions -------------------------------------------------------------------------------------------------------
def rotate_neighbours(x, dims, base):
    """x [L, heads, D]: the pairs (2i, 2i + 1), i < dims / 2, turned by position * base^(-2i / dims)."""
    L = x.shape[0]
    out = x.clone()
    pos = torch.arange(L, dtype=torch.float64)
    for i in range(dims // 2):
        a = pos * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a).to(x.dtype)[:, None], torch.sin(a).to(x.dtype)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def query_temperature(L, coef, every):
    """One factor per position: 1 + coef ln(floor((p + 1) / every) + 1)."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in range(L)], dtype=torch.float64)


def distance_bucket(n, rows, far):
    """Distances below rows / 2 have a row each; the rest share the other half in logarithmic steps up to ``far``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def distance_bias(L, table, far):
    """[H, L, L]: table[bucket(i - j), h] for j <= i (zero above the diagonal, where nothing is visible)."""
    rows, H = table.shape
    out = torch.zeros(H, L, L, dtype=table.dtype)
    for i in range(L):
        for j in range(i + 1):
            out[:, i, j] = table[distance_bucket(i - j, rows, far)]
    return out


def visible(L, window=None):
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


def softmax_with_extra(s, ok, extra=None):
    """Softmax over the visible keys; ``extra`` [H] joins the denominator as exp(extra) without key or value."""
    s = s.masked_fill(~ok, float("-inf"))
    m = s.max(-1, keepdim=True).values
    if extra is not None:
        m = torch.maximum(m, extra.reshape(-1, 1, 1))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if extra is not None:
        den = den + torch.exp(extra.reshape(-1, 1, 1) - m)
    return e / den


# ---- mixers ----------------------------------------------------------------------------------------------------------
def _qkv(h, w, m, eps):
    L = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).reshape(L, H, D)
    k = (h @ w["k"].T + w["k.b"]).reshape(L, G, D)
    v = (h @ w["v"].T + w["v.b"]).reshape(L, G, E)
    return unit_rms(q, eps) * w["q.norm"], unit_rms(k, eps) * w["k.norm"], v


def _mix_values(v, w, m, shared):
    """The first layer that mixes values keeps its own and lends them to the later ones."""
    if not m.get("v_mix"):
        return v
    if "v_first" not in shared:
        shared["v_first"] = v
        return v
    lam = w["vmix"]
    return (1 - lam) * v + lam * shared["v_first"].reshape(v.shape)          # rows of equal width, whatever the heads


def _attend(q, k, v, s_fn, ok, extra):
    """q [L, H, D], k [L, G, D], v [L, G, E] -> [L, H * E]; s_fn maps raw dot products [H, L, L] to scores."""
    L, H, _ = q.shape
    G = k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    vv = v.repeat_interleave(H // G, dim=1)
    s = s_fn(torch.einsum("ihd,jhd->hij", q, kk))
    p = softmax_with_extra(s, ok, extra)
    return torch.einsum("hij,jhe->ihe", p, vv).reshape(L, -1)


def biased_attention(h, w, m, eps, shared):
    """No rotation; queries grow with the logarithm of their position, a learned bias per distance bucket and head
    joins the score, the softmax's denominator holds one more 1, and a sigmoid gate multiplies the heads' outputs."""
    L = h.shape[0]
    H = m["heads"]
    q, k, v = _qkv(h, w, m, eps)
    t = m.get("q_temp")
    if t:
        q = q * query_temperature(L, t["coef"], t["every"]).to(q.dtype)[:, None, None]
    v = _mix_values(v, w, m, shared)
    bias = distance_bias(L, w["rel"], m["bias_max"])
    o = _attend(q, k, v, lambda d: d * m["scale"] + bias, visible(L), torch.zeros(H, dtype=h.dtype))
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def capped_window_attention(h, w, m, eps, shared):
    """Part-rotated heads (neighbouring pairs), scores squashed by cap * tanh(score / cap), a sliding window."""
    L = h.shape[0]
    q, k, v = _qkv(h, w, m, eps)
    rot = m.get("rot")
    if rot:
        q, k = rotate_neighbours(q, rot["dims"], rot["base"]), rotate_neighbours(k, rot["dims"], rot["base"])
    v = _mix_values(v, w, m, shared)
    cap = m.get("softcap")

    def score(d):
        d = d * m["scale"]
        return cap * torch.tanh(d / cap) if cap else d
    o = _attend(q, k, v, score, visible(L, (m.get("mask") or {}).get("size")), None)
    return o @ w["o"].T


def latent_attention(h, w, m, eps, shared):
    """Queries through a normed latent; keys and values from one normed latent per token plus a rotated key part that
    all heads share; one learned number per head joins the softmax's denominator."""
    L = h.shape[0]
    H, D, P, E, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = unit_rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(L, H, D + P)
    down = h @ w["dkv"].T
    c = unit_rms(down[:, :R], eps) * w["dkv.norm"]
    base = m["rot"]["base"]
    k_rot = rotate_neighbours(down[:, None, R:], P, base)                 # [L, 1, P]
    q_rot = rotate_neighbours(q[..., D:], P, base)
    k = torch.cat([(c @ w["uk"].T).reshape(L, H, D), k_rot.expand(L, H, P)], dim=-1)
    v = (c @ w["uv"].T).reshape(L, H, E)
    q = torch.cat([q[..., :D], q_rot], dim=-1)
    o = _attend(q, k, v, lambda d: d * m["scale"], visible(L), w["sink"])
    return o @ w["o"].T


MIXERS = {"attention": biased_attention, "attention_2": capped_window_attention, "latent_attention": latent_attention}


# ---- feed-forward ------------------------------------------------------------------------------------------------------
def gated_ff(h, w):
    g = h @ w["gate"].T
    return (g * torch.sigmoid(g) * (h @ w["up"].T)) @ w["down"].T


def route(h, w, r):
    """Returns (chosen [L, top], weights [L, top]) over experts + identity slots."""
    n = r["experts"] + r.get("identity", 0)
    s = torch.softmax(h.double() @ w["router"].double().T, dim=-1)
    choice = s + w["correction"].double()
    groups = r.get("groups")
    if groups and groups["count"] > 1:
        per = n // groups["count"]
        best = choice.reshape(-1, groups["count"], per).max(-1).values
        kept = best.topk(groups["keep"], dim=-1).indices
        allow = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(per, dim=1)
        choice = choice.masked_fill(~allow, float("-inf"))
    idx = choice.topk(r["top"], dim=-1).indices
    wts = s.gather(1, idx)
    return idx, (wts / (wts.sum(-1, keepdim=True) + 1e-20)).to(h.dtype)


def moe(h, w, mlp):
    r = mlp["router"]
    idx, wts = route(h, w, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wts[t]):
            if e >= r["experts"]:
                out[t] += a * h[t]                                             # an identity slot: the input itself
            else:
                out[t] += a * gated_ff(h[t:t + 1], sub(w, f"e{e}."))[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, sub(w, "shared."))
    return out


# ---- the stack -------------------------------------------------------------------------------------------------------
def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, dtype=torch.float32, want_layers=False):
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    x = W["embed"][torch.tensor(tokens)]
    trail, shared = [], {}
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = group_norm(x, W[p + "norm1"], groups, eps)
        y = MIXERS[spec["type"]](h, sub(W, p + "mix."), spec["mixer"], eps, shared)
        y = y * W[p + "ls1"] * torch.sigmoid(h @ W[p + "rg1"].T + W[p + "rg1.b"])
        if spec.get("mlp") is not None:
            f = moe(h, sub(W, p + "mlp."), spec["mlp"])
            y = y + f * W[p + "ls2"] * torch.sigmoid(h @ W[p + "rg2"].T + W[p + "rg2.b"])
        x = x + y
        trail.append(x)
    logits = group_norm(x, W["final.norm"], groups, eps) @ W["head"].T
    return (logits, torch.stack(trail)) if want_layers else logits


# ---- small models ----------------------------------------------------------------------------------------------------
def feed_forward(ff=40, experts=6, top=2, identity=2, groups=(2, 1), shared=24):
    r = {"experts": experts, "top": top}
    if identity:
        r["identity"] = identity
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def _mlp(mlp):
    return feed_forward() if mlp == "moe" else mlp


def bias_layer(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.3, bias_max=40, q_temp=(0.4, 7), v_mix=False, mlp="moe"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": _mlp(mlp)}


def cap_layer(heads=4, kv_heads=2, dim=12, vdim=20, window=9, rot_dims=8, base=100.0, scale=0.3, softcap=4.0,
              v_mix=False, mlp="moe"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    if softcap:
        m["softcap"] = softcap
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention_2", "mixer": m, "mlp": _mlp(mlp)}


def latent_layer(heads=3, dim=12, rot_dim=8, vdim=20, kv_rank=24, q_rank=16, base=100.0, scale=0.3, mlp="moe"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale, "rot": {"base": base, "dims": rot_dim}}
    return {"type": "latent_attention", "mixer": m, "mlp": _mlp(mlp)}


def make_config(layers, vocab=96, width=48, eps=1e-5, groups=4):
    return {"architecture": "Lefolorn", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups},
            "layers": layers}


def make_weights(cfg, seed=0, dtype=torch.bfloat16, rows=10):
    """``rows``: distance buckets of the biased layers (a number, or one per layer index)."""
    g = torch.Generator().manual_seed(seed)
    Wd = cfg["width"]

    def lin(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * gain / i ** 0.5

    def vec(n, mean=0.0, spread=0.1):
        return mean + spread * torch.randn(n, generator=g)
    W = {"embed": torch.randn(cfg["vocab"], Wd, generator=g), "final.norm": vec(Wd, 1.0),
         "head": lin(cfg["vocab"], Wd, 2.0)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        W[p + "norm1"] = vec(Wd, 1.0, 0.2)
        W[p + "ls1"], W[p + "ls2"] = vec(Wd, 0.8, 0.3), vec(Wd, 0.8, 0.3)
        for n in ("rg1", "rg2"):
            W[p + n], W[p + n + ".b"] = lin(Wd, Wd, 2.0), vec(Wd, 0.5, 0.5)
        H, E = m["heads"], m["vdim"]
        if spec["type"] == "latent_attention":
            D, P, R, Q = m["dim"], m["rot_dim"], m["kv_rank"], m["q_rank"]
            W[p + "mix.dq"], W[p + "mix.dq.norm"] = lin(Q, Wd, 2.0), vec(Q, 1.0, 0.2)
            W[p + "mix.uq"] = lin(H * (D + P), Q, 2.0)
            W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = lin(R + P, Wd, 2.0), vec(R, 1.0, 0.2)
            W[p + "mix.uk"], W[p + "mix.uv"] = lin(H * D, R, 2.0), lin(H * E, R)
            W[p + "mix.sink"] = vec(H, 0.5, 1.0)
        else:
            G, D = m["kv_heads"], m["dim"]
            for n, r_ in (("q", H * D), ("k", G * D), ("v", G * E)):
                W[p + "mix." + n] = lin(r_, Wd, 2.0)
                W[p + "mix." + n + ".b"] = vec(r_, 0.0, 0.3)
            W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(D, 1.0, 0.2), vec(D, 1.0, 0.2)
            if m.get("v_mix"):
                W[p + "mix.vmix"] = vec((), 0.4, 0.2)
            if spec["type"] == "attention":
                n_rows = rows[i] if isinstance(rows, dict) else rows
                W[p + "mix.rel"] = torch.randn(n_rows, H, generator=g) * 1.5
                W[p + "mix.g"] = lin(H * E, Wd, 2.0)
        W[p + "mix.o"] = lin(Wd, H * E)
        mlp = spec.get("mlp")
        if mlp is None:
            del W[p + "ls2"], W[p + "rg2"], W[p + "rg2.b"]
            continue
        r = mlp["router"]
        n = r["experts"] + r.get("identity", 0)
        W[p + "mlp.router"] = lin(n, Wd, 3.0)
        W[p + "mlp.correction"] = vec(n, -0.1, 0.15)                         # choice scores of both signs
        for e in range(r["experts"]):
            W[p + f"mlp.e{e}.gate"] = lin(mlp["expert"]["ff"], Wd, 1.5)
            W[p + f"mlp.e{e}.up"] = lin(mlp["expert"]["ff"], Wd, 1.5)
            W[p + f"mlp.e{e}.down"] = lin(Wd, mlp["expert"]["ff"])
        if mlp.get("shared"):
            W[p + "mlp.shared.gate"] = lin(mlp["shared"]["ff"], Wd, 1.5)
            W[p + "mlp.shared.up"] = lin(mlp["shared"]["ff"], Wd, 1.5)
            W[p + "mlp.shared.down"] = lin(Wd, mlp["shared"]["ff"])
    return {k: v.to(dtype) for k, v in W.items()}


def save_checkpoint(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def logit_error(got, want):
    """Root mean square of the difference (its mean over the vocabulary taken off), relative to the spread of the
    wanted logits."""
    d = got.float() - want.float()
    d = d - d.mean(-1, keepdim=True)
    spread = (want.float() - want.float().mean(-1, keepdim=True)).pow(2).mean().sqrt()
    return (d.pow(2).mean().sqrt() / spread).item()
