"""A slow, whole-sequence implementation of the Sevazen design, one function per mechanism, written from its equations
and sharing no code with the package: the oracle of tests/test_sevazen.py.  Everything runs in fp32 (or fp64) on the
CPU over one whole sequence at a time; there is no cache, no batching and no portioning here.

Notation: x residual [L, W]; a layer computes x <- x + LN_1(mixer(x)), then x <- x + LN_2(ff(x)).
"""
import json
import math
import os

import torch


# ---- norms ---------------------------------------------------------------------------------------------------------
def layer_norm(y, w, b, eps):
    mu = y.mean(-1, keepdim=True)
    var = ((y - mu) ** 2).mean(-1, keepdim=True)
    return (y - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(y, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


# ---- short causal convolution ----------------------------------------------------------------------------------------
def short_conv(u, w):
    """u [L, C], w [C, taps]:  y[t] = sum_j w[:, j] u[t - taps + 1 + j], zeros before the sequence."""
    L, C = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u])
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + w[:, j] * padded[j: j + L]
    return y


# ---- rotation --------------------------------------------------------------------------------------------------------
def base_freqs(rot):
    n = rot["dims"] // 2
    return torch.tensor([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(n)], dtype=torch.float64)


def freqs_by_wavelength(rot):
    """Short waves keep their frequency, long ones are slowed by ``factor``, a blend between (returns f, magnitude)."""
    f = base_freqs(rot)
    s = rot.get("scaling")
    if not s:
        return f, 1.0
    out = []
    for fi in f.tolist():
        wave = 2 * math.pi / fi
        if wave < s["original"] / s["high"]:
            out.append(fi)
        elif wave > s["original"] / s["low"]:
            out.append(fi / s["factor"])
        else:
            t = (s["original"] / wave - s["low"]) / (s["high"] - s["low"])
            out.append((1 - t) * fi / s["factor"] + t * fi)
    return torch.tensor(out, dtype=torch.float64), 1.0


def freqs_by_ramp(rot):
    """A ramp over the pair index decides how much of the slowed frequency each pair takes; cos and sin are stretched."""
    f = base_freqs(rot)
    s = rot.get("scaling")
    if not s:
        return f, 1.0
    dims, base = rot["dims"], rot["base"]

    def index_of(turns):
        return dims * math.log(s["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(index_of(s["fast"])), 0)
    hi = min(math.ceil(index_of(s["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f.tolist()):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / s["factor"] * r + fi * (1 - r))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(s["factor"]) + 1.0


def rotate(x, freqs, magnitude, dims):
    """x [L, heads, D]: value i < dims / 2 and value i + dims / 2 form a pair, turned by position * freqs[i]."""
    if dims == 0:
        return x
    L = x.shape[0]
    ang = torch.arange(L, dtype=torch.float64)[:, None] * freqs[None, :]
    c = (torch.cos(ang) * magnitude).to(x.dtype)[:, None, :]
    s = (torch.sin(ang) * magnitude).to(x.dtype)[:, None, :]
    a, b = x[..., : dims // 2], x[..., dims // 2: dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


# ---- mixers ------------------------------------------------------------------------------------------------------------
def project(h, w, name):
    y = h @ w[name].T
    return y + w[name + ".b"] if name + ".b" in w else y


def visible(L, window=None, chunk=None):
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    if chunk:
        ok = ok & (i // chunk == j // chunk)
    return ok


def sink_window_attention(h, w, m, eps):
    """Grouped-query attention: biased projections, short convolution, q / k norms, part rotation, a sliding window and
    a sink in the denominator."""
    L = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = project(h, w, "q"), project(h, w, "k"), project(h, w, "v")
    if m.get("conv"):
        q, k, v = short_conv(q, w["q.conv"]), short_conv(k, w["k.conv"]), short_conv(v, w["v.conv"])
    q = unit_rms(q.view(L, H, D), eps) * w["q.norm"]
    k = unit_rms(k.view(L, G, D), eps) * w["k.norm"]
    v = v.view(L, G, E)
    rot = m.get("rot")
    if rot:
        f, mag = freqs_by_wavelength(rot)
        q, k = rotate(q, f, mag, rot["dims"]), rotate(k, f, mag, rot["dims"])
    ok = visible(L, window=(m.get("mask") or {}).get("size"))
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~ok, float("-inf"))
        shift = torch.maximum(s.max(-1, keepdim=True).values, w["sink"][a])
        e = torch.exp(s - shift)
        den = e.sum(-1, keepdim=True) + torch.exp(w["sink"][a] - shift)        # the sink: in the sum, no value
        heads.append((e / den) @ v[:, g])
    return torch.cat(heads, -1) @ w["o"].T


def differential_chunk_attention(h, w, m, eps):
    """Two score maps per head over the same values, keys of the query's own chunk only, o = a1 - lambda a2, normed per
    head, gated."""
    L = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms(project(h, w, "q").view(L, H, 2, D), eps) * w["q.norm"]
    k = unit_rms(project(h, w, "k").view(L, G, 2, D), eps) * w["k.norm"]
    v = project(h, w, "v").view(L, G, E)
    rot = m.get("rot")
    if rot:
        f, mag = freqs_by_ramp(rot)
        q = rotate(q.reshape(L, 2 * H, D), f, mag, rot["dims"]).view(L, H, 2, D)
        k = rotate(k.reshape(L, 2 * G, D), f, mag, rot["dims"]).view(L, G, 2, D)
    ok = visible(L, chunk=(m.get("mask") or {}).get("size"))
    lam = torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + m["diff"]
    heads = []
    for a in range(H):
        g = a // (H // G)
        maps = []
        for c in range(2):
            s = (q[:, a, c] @ k[:, g, c].T) * m["scale"]
            maps.append(torch.softmax(s.masked_fill(~ok, float("-inf")), -1) @ v[:, g])
        heads.append(unit_rms(maps[0] - lam * maps[1], eps) * (1 - m["diff"]))
    o = torch.cat(heads, -1) * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


MIXERS = {"attention": sink_window_attention, "attention_2": differential_chunk_attention}


# ---- feed-forwards ---------------------------------------------------------------------------------------------------
def squared_relu_ff(h, w):
    return torch.relu(h @ w["up"].T) ** 2 @ w["down"].T


def route(h, w, r):
    """The ``top`` largest router logits and the softmax over just those."""
    z = h @ w["router"].T + w["router.b"]
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    val, idx = val[:, : r["top"]], idx[:, : r["top"]]
    return torch.softmax(val, -1), idx


def moe(h, w, mlp):
    weight, idx = route(h, w, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(idx.shape[1]):
            e = int(idx[t, c])
            out[t] += weight[t, c] * squared_relu_ff(h[t: t + 1], sub(w, f"e{e}."))[0]
    if mlp.get("shared"):
        out = out + squared_relu_ff(h, sub(w, "shared.")) * torch.sigmoid(h @ w["shared.sg"].T)
    return out


# ---- the stack -------------------------------------------------------------------------------------------------------
def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def owner(cfg, i):
    while cfg["layers"][i].get("weights_of") is not None:
        i = cfg["layers"][i]["weights_of"]
    return i


def forward(cfg, weights, tokens, dtype=torch.float32, want_layers=False):
    W = {k: v.to(dtype) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    trail = []
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{owner(cfg, i)}."
        y = MIXERS[spec["type"]](x, sub(W, p + "mix."), spec["mixer"], eps)
        x = x + layer_norm(y, W[p + "norm1"], W[p + "norm1.b"], eps)
        mlp = spec.get("mlp")
        if mlp is not None:
            y = squared_relu_ff(x, sub(W, p + "mlp.")) if mlp["kind"] == "dense" else moe(x, sub(W, p + "mlp."), mlp)
            x = x + layer_norm(y, W[p + "norm2"], W[p + "norm2.b"], eps)
        trail.append(x)
    logits = layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["embed"].T
    return (logits, torch.stack(trail)) if want_layers else logits


# ---- small models ----------------------------------------------------------------------------------------------------
def feed_forward(kind, ff=40, experts=6, top=2, shared=24):
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": ff}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def _mlp(mlp):
    return feed_forward(mlp) if mlp is None or isinstance(mlp, str) else mlp


def window_layer(heads=4, kv_heads=2, dim=12, vdim=20, window=9, conv=3, rot_dims=8, base=100.0, scale=0.3,
                 scaling=(4.0, 1.0, 4.0, 16), mlp="moe", weights_of=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if conv:
        m["conv"] = conv
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    d = {"type": "attention", "mixer": m, "mlp": _mlp(mlp)}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def diff_layer(heads=2, kv_heads=1, dim=8, vdim=12, chunk=11, rot_dims=4, base=50.0, scale=0.4, diff=0.3,
               scaling=(2.0, 24, 8.0, 1.0), mlp="dense", weights_of=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if chunk:
        m["mask"] = {"size": chunk}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    d = {"type": "attention_2", "mixer": m, "mlp": _mlp(mlp)}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def make_config(layers, vocab=96, width=48, eps=1e-5):
    return {"architecture": "Sevazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def make_weights(cfg, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    Wd = cfg["width"]

    def lin(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * gain / i ** 0.5

    def vec(n, mean=0.0, spread=0.1):
        return mean + spread * torch.randn(n, generator=g)
    W = {"embed": torch.randn(cfg["vocab"], Wd, generator=g), "final.norm": vec(Wd, 1.0), "final.norm.b": vec(Wd)}
    for i, spec in enumerate(cfg["layers"]):
        if spec.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", spec["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        maps = 2 if spec["type"] == "attention_2" else 1
        W[p + "norm1"], W[p + "norm1.b"] = vec(Wd, 1.0), vec(Wd)
        for n, rows in (("q", H * maps * D), ("k", G * maps * D), ("v", G * E)):
            W[p + "mix." + n] = lin(rows, Wd, 2.0)
            W[p + "mix." + n + ".b"] = vec(rows, 0.0, 0.3)
            if m.get("conv"):
                W[p + f"mix.{n}.conv"] = torch.randn(rows, m["conv"], generator=g) * 0.6
        W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(D, 1.0, 0.2), vec(D, 1.0, 0.2)
        W[p + "mix.o"] = lin(Wd, H * E)
        if maps == 1:
            W[p + "mix.sink"] = vec(H, 0.5, 1.0)
        else:
            for n in ("lq1", "lk1", "lq2", "lk2"):
                W[p + "mix." + n] = vec(D, 0.0, 0.5 / D ** 0.25)          # their dot products: about +- 0.25
            W[p + "mix.g"] = lin(H * E, Wd, 2.0)
        mlp = spec.get("mlp")
        if mlp is None:
            continue
        W[p + "norm2"], W[p + "norm2.b"] = vec(Wd, 1.0), vec(Wd)
        if mlp["kind"] == "dense":
            W[p + "mlp.up"], W[p + "mlp.down"] = lin(mlp["ff"], Wd, 1.5), lin(Wd, mlp["ff"])
        else:
            E_ = mlp["router"]["experts"]
            W[p + "mlp.router"], W[p + "mlp.router.b"] = lin(E_, Wd, 3.0), vec(E_, 0.0, 0.5)
            for e in range(E_):
                W[p + f"mlp.e{e}.up"] = lin(mlp["expert"]["ff"], Wd, 1.5)
                W[p + f"mlp.e{e}.down"] = lin(Wd, mlp["expert"]["ff"])
            if mlp.get("shared"):
                W[p + "mlp.shared.up"] = lin(mlp["shared"]["ff"], Wd, 1.5)
                W[p + "mlp.shared.down"] = lin(Wd, mlp["shared"]["ff"])
                W[p + "mlp.shared.sg"] = lin(1, Wd, 2.0)
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
