"""Lefolorn (parallel sub-layers behind per-channel gates over an fp32 residual normed in groups; softmax attention with
a distance-bias table, a query temperature, one more 1 in the denominator and an output gate; soft-capped window
attention with neighbour-paired rotation; value mixing across layers; latent attention with a query latent and learned
sinks; softmax group-limited routing with identity experts and a shared expert) against the slow oracle of
tests/lefolorn_oracle.py: every mechanism alone, then whole models through the engine's own scheduler, page pool and
step function -- on the CPU backend (fp32) and, marked gpu, through the HIP kernels (fp32 and bf16).  Small random
models are written to disk as checkpoints, so the loader and the configuration reader run too."""
import pytest
import torch

import lefolorn_oracle as O
from vllm_distributed_amd import ops

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
OP_CASES = [("cpu", torch.float32), pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
            pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]
# 16-bit: models this narrow (48 values per row) average little rounding away; the crafted cases move by O(1)
TOL = {"float32": 2e-4, "bfloat16": 0.25}
OP_TOL = {torch.float32: 3e-5, torch.bfloat16: 2.5e-2}


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(0)


def rel(got, want):
    got, want = got.float().cpu(), want.float().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-20)).item()


def mixed_layers():
    """All three mixers; values mixed across the two attention kinds; one layer without a feed-forward."""
    return [O.latent_layer(), O.bias_layer(v_mix=True), O.cap_layer(v_mix=True),
            O.bias_layer(heads=6, kv_heads=2, dim=8, vdim=20, v_mix=True, q_temp=(0.7, 3), mlp=None),
            O.latent_layer(heads=2, dim=6, rot_dim=12, vdim=10, kv_rank=20, q_rank=9,
                           mlp=O.feed_forward(experts=7, top=3, identity=2, groups=(3, 2), shared=None))]


def matrix_core_layers():
    """Widths the matrix-core kernels take in 16-bit runs (keys and values of 64 / 128 alike; latent rows of 64 + 32
    and 128 + 32); other runs take the kernels for any sizes."""
    return [O.latent_layer(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64, q_rank=24, mlp="moe"),
            O.cap_layer(heads=4, kv_heads=2, dim=64, vdim=64, window=21, rot_dims=32, v_mix=True, mlp=None),
            O.bias_layer(heads=4, kv_heads=2, dim=64, vdim=64, bias_max=30, v_mix=True, mlp="moe"),
            O.bias_layer(heads=2, kv_heads=1, dim=128, vdim=128, bias_max=23, q_temp=(0.3, 16), v_mix=True, mlp=None),
            O.latent_layer(heads=2, dim=24, rot_dim=32, vdim=8, kv_rank=128, q_rank=40, mlp=None)]


LAYER_SETS = {"mixed": mixed_layers, "matrix_core": matrix_core_layers}


# ---- driving the engine ------------------------------------------------------------------------------------------
def run_schedule(folder, dtype, device, prompts, schedule, max_tokens, block_size=16, eager=True):
    """``schedule``: steps of (request, token count); every request ends when its tokens are used up.  Returns
    request -> logits [tokens, vocab] in the order the tokens ran."""
    from vllm_distributed_amd.entrypoints.trace_replay import TraceReplayer
    r = TraceReplayer(folder, dtype, max_tokens, block_size=block_size, device=device, enforce_eager=eager)
    at = {k: 0 for k in prompts}
    got = {k: [] for k in prompts}
    try:
        for step in schedule:
            entries, end = [], []
            for rid, n in step:
                lo, hi = at[rid], at[rid] + n
                entries.append({"id": rid, "tokens": prompts[rid][lo:hi], "want": list(range(n))})
                at[rid] = hi
                if hi == len(prompts[rid]):
                    end.append(rid)
            rows = torch.from_numpy(r.step(entries, end))
            o = 0
            for rid, n in step:
                got[rid].append(rows[o:o + n])
                o += n
    finally:
        r.shutdown()
    assert all(at[k] == len(prompts[k]) for k in prompts)
    return {k: torch.cat(v) for k, v in got.items()}


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def check(cfg, W, prompts, got, dtype):
    """Every position within the tolerance.  The exception: 16-bit runs of models with routed experts.  There a choice
    that is a close call in the oracle can fall the other way under rounding, which moves that position by O(1); such
    runs bound the typical error and the share of positions beyond the tolerance instead (the fp32 runs of the same
    kernels stay exact position by position)."""
    routed = any(l.get("mlp") is not None for l in cfg["layers"])
    for rid, p in prompts.items():
        want = O.forward(cfg, W, p)
        if dtype == "bfloat16" and routed:
            errs = torch.tensor([O.logit_error(got[rid][i], want[i]) for i in range(len(p))])
            assert errs.median() < TOL[dtype] / 2 and (errs > TOL[dtype]).float().mean() <= 0.3 and errs.max() < 1.0, \
                f"request {rid}: median error {errs.median():.2e}, {(errs > TOL[dtype]).sum()} of {len(p)} beyond"
            continue
        err = O.logit_error(got[rid], want)
        assert err < TOL[dtype], f"request {rid}: logits differ by {err:.2e} of their spread"


def model(tmp_path, layers, seed=0, rows=10, **kw):
    cfg = O.make_config(layers, **kw)
    W = O.make_weights(cfg, seed, rows=rows)
    return O.save_checkpoint(str(tmp_path / "m"), cfg, W), cfg, W


def pages(lens, bs, spare=3):
    """Scattered pages for sequences of the given lengths: (block table, number of blocks)."""
    nblk = sum(-(-n // bs) for n in lens) + spare
    perm = torch.randperm(nblk - 1) + 1
    table = torch.zeros(len(lens), max(-(-n // bs) for n in lens), dtype=torch.int32)
    o = 0
    for s, n in enumerate(lens):
        k = -(-n // bs)
        table[s, :k] = perm[o:o + k].int()
        o += k
    return table, nblk


# ---- mechanisms alone ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dev,dt", OP_CASES)
@pytest.mark.parametrize("W_,groups", [(48, 4), (300, 3), (33, 1), (512, 8), (70, 7), (512, 2), (1024, 4), (3072, 3),
                                       (4096, 2), (1280, 5), (1024, 8), (2048, 64), (64, 4), (1536, 12)])
def test_gated_parallel_residual_with_group_norm(dev, dt, W_, groups):
    T, eps = 7, 1e-5
    x = torch.randn(T, W_) * 3 + 1
    y1, y2, g1, g2, h = [(torch.randn(T, W_ + 4) * 2).to(dt)[:, :W_] for _ in range(5)]
    s1, s2, w = 1 + 0.3 * torch.randn(W_), 0.5 * torch.randn(W_), 1 + 0.2 * torch.randn(W_)
    idw = torch.rand(T)

    def d(t):
        return t.to(dev) if t is not None else None
    # first norm of a stack: nothing joins x
    xd = x.clone().to(dev)
    first = ops.gated_residual_group_norm(xd, [], d(w), groups, eps, dt)
    torch.testing.assert_close(xd.cpu(), x)
    assert first.dtype == dt and rel(first, O.group_norm(x, w, groups, eps)) < OP_TOL[dt]
    # one sub-layer, then two with an identity share of the second's input
    for subs, want in (
            ([(y1, s1, g1, None, None)], x + y1.float() * s1 * torch.sigmoid(g1.float())),
            ([(y1, s1, g1, None, None), (y2, s2, g2, h, idw)],
             x + (y1.float() * s1 * torch.sigmoid(g1.float())
                  + (y2.float() + idw[:, None] * h.float()) * s2 * torch.sigmoid(g2.float()))),
            ([(y1, None, None, None, None), (y2, s2, None, None, None)], x + (y1.float() + y2.float() * s2)),
            ([(y1, s1, g1, None, None), (y2, s2, g2, h, idw), (g1, s2, g2, None, None)],
             x + (y1.float() * s1 * torch.sigmoid(g1.float())
                  + (y2.float() + idw[:, None] * h.float() + g1.float()) * s2 * torch.sigmoid(g2.float())))):
        xd = x.clone().to(dev)
        nxt = ops.gated_residual_group_norm(xd, [tuple(d(t) for t in sub) for sub in subs], d(w), groups, eps, dt)
        torch.testing.assert_close(xd.cpu(), want, atol=3e-5, rtol=1e-5)
        assert rel(nxt, O.group_norm(want, w, groups, eps)) < OP_TOL[dt]
    xd = x.clone().to(dev)                                 # the last update of a stack that ends without a norm
    assert ops.gated_residual_group_norm(xd, [(d(y1), d(s1), None, None, None)], None, groups, eps, dt) is None
    torch.testing.assert_close(xd.cpu(), x + y1.float() * s1, atol=3e-5, rtol=1e-5)


def test_distance_buckets_against_the_oracle():
    from vllm_distributed_amd.layers.masked_attention import log_bucket_rows
    for rows, far in ((10, 40), (16, 200), (4, 9), (32, 257), (7, 30), (2, 5)):
        got = log_bucket_rows(rows, far).tolist()
        assert got == [O.distance_bucket(n, rows, far) for n in range(far + 1)]
        assert got[-1] == rows - 1 == O.distance_bucket(far + 1000, rows, far)
        assert got[: rows // 2] == list(range(rows // 2)) and sorted(got) == got


@pytest.mark.parametrize("dev,dt", OP_CASES)
@pytest.mark.parametrize("n,ident,top,groups,keep", [(8, 2, 2, 2, 1), (9, 0, 3, 3, 2), (6, 1, 1, 1, 1), (12, 3, 4, 4, 3),
                                                     (70, 6, 5, 7, 2), (5, 5, 2, 1, 1)])
def test_group_limited_softmax_choice_with_identity_outputs(dev, dt, n, ident, top, groups, keep):
    """Choice scores of both signs (groups that are out count as minus infinity, not zero), the plain scores as weights
    divided by their sum, winners without an expert reported apart."""
    from vllm_distributed_amd.layers.moe import grouped_topk_with_identity
    T, Wd = 50, 24
    x = torch.randn(T, Wd)
    w = {"router": torch.randn(n, Wd) * 0.7, "correction": -0.2 + 0.2 * torch.randn(n)}
    r = {"experts": n - ident, "identity": ident, "top": top, "groups": {"count": groups, "keep": keep}}
    want_ids, want_w = O.route(x, w, r)
    logits = (x @ w["router"].T).to(dev)
    tw, ids, idw = grouped_topk_with_identity(logits, w["correction"].to(dev), top, groups, keep, True, "softmax",
                                              "max", ident, 1e-20)
    tw, ids = tw.cpu(), ids.cpu().long()
    is_id = want_ids >= n - ident
    assert torch.equal(ids.clamp_min(-1).sort(-1).values, want_ids.masked_fill(is_id, -1).sort(-1).values)
    real = want_w.float().masked_fill(is_id, 0.0)
    torch.testing.assert_close(tw.gather(1, ids.argsort(-1)), real.gather(1, want_ids.masked_fill(is_id, -1).argsort(-1)),
                               atol=1e-5, rtol=1e-4)
    if ident:
        torch.testing.assert_close(idw.cpu(), (want_w.float() * is_id).sum(-1), atol=1e-5, rtol=1e-4)
        assert is_id.any()
    else:
        assert idw is None


@pytest.mark.parametrize("dev,dt", OP_CASES)
@pytest.mark.parametrize("Wd,ff,E,ident,top,T", [(24, 10, 5, 1, 2, 9), (33, 7, 3, 2, 3, 4), (48, 80, 6, 0, 3, 70),
                                                 (256, 128, 8, 2, 2, 150), (128, 64, 4, 4, 2, 3),
                                                 (256, 128, 8, 2, 2, 1300)])
def test_gated_experts_with_identity_choices(dev, dt, Wd, ff, E, ident, top, T):
    """The experts' weighted sum when some winners have no expert (their share is the input itself); the last sizes are
    ones the matrix-core expert kernels take in 16-bit (few pairs: the grouped skinny form, many: the tiled form)."""
    from vllm_distributed_amd.layers.moe import grouped_topk_with_identity
    if T > 1000 and dev == "cpu":
        pytest.skip("the tiled form is a device kernel")
    x = torch.randn(T, Wd).to(dt)
    n = E + ident
    w = {"router": torch.randn(n, Wd) / Wd ** 0.5 * 3, "correction": 0.05 * torch.randn(n)}
    for e in range(E):
        w[f"e{e}.gate"] = (torch.randn(ff, Wd) / Wd ** 0.5 * 1.5).to(dt).float()
        w[f"e{e}.up"] = (torch.randn(ff, Wd) / Wd ** 0.5 * 1.5).to(dt).float()
        w[f"e{e}.down"] = (torch.randn(Wd, ff) / ff ** 0.5).to(dt).float()
    mlp = {"router": {"experts": E, "identity": ident, "top": top}}
    want = O.moe(x.float(), w, mlp)
    logits = (x.float() @ w["router"].T).to(dev)
    tw, ids, idw = grouped_topk_with_identity(logits, w["correction"].to(dev), top, 1, 1, True, "softmax", "max", ident,
                                              1e-20)
    w13 = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).to(dt).to(dev)
    w2 = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(dt).to(dev)
    got = ops.fused_moe(x.to(dev), w13, w2, tw, ids, activation="silu").float().cpu()
    if ident:
        got = got + idw.cpu()[:, None] * x.float()
    assert rel(got, want) < OP_TOL[dt]


def selection(rows, lo, n):
    """[n, rows]: picks columns lo .. lo + n of a row."""
    m = torch.zeros(n, rows)
    m[torch.arange(n), lo + torch.arange(n)] = 1.0
    return m


# (heads, kv heads, D, Dv, kind, window, soft cap, (bucket rows, far), (coef, every), rotated dims, values mixed)
ATTN_SIZES = [
    (4, 2, 12, 20, "bias", 0, 0.0, (10, 40), (0.4, 7), 0, True), (4, 2, 12, 20, "cap", 9, 4.0, None, None, 8, True),
    (6, 3, 64, 64, "cap", 37, 2.5, None, None, 16, False), (6, 3, 64, 64, "bias", 0, 0.0, (8, 21), (1.0, 1), 0, False),
    (3, 3, 5, 7, "bias", 0, 0.0, (3, 70), None, 0, False), (1, 1, 4, 2, "cap", 1, 0.0, None, None, 4, False),
    (8, 1, 16, 16, "cap", 33, 9.0, None, None, 16, True), (8, 2, 128, 128, "bias", 0, 0.0, (32, 64), (0.2, 50), 0, True),
    (8, 2, 128, 128, "cap", 30, 6.0, None, None, 64, True), (2, 1, 96, 96, "cap", 0, 1.5, None, None, 0, False),
    (12, 2, 64, 64, "bias", 0, 0.0, (16, 33), None, 0, True), (2, 2, 32, 8, "cap", 70, 3.0, None, None, 24, False)]


@pytest.mark.parametrize("dev,dt", OP_CASES)
@pytest.mark.parametrize("H,G,D,E,kind,window,cap,dist,temp,rot,vmix", ATTN_SIZES)
@pytest.mark.parametrize("bs", [16, 32])
def test_attention_paged(dev, dt, H, G, D, E, kind, window, cap, dist, temp, rot, vmix, bs):
    """Ragged batch on scattered pages -- a single decoded token, a portion of a prompt behind cached context that
    starts inside a page, a whole prompt -- against the oracle's dense computation per sequence; contexts longer than
    windows and bias tables, so that hidden and far keys sit in pages of their own.  The bias table's rows differ by
    O(1), so a key in the wrong bucket shows."""
    paged_case(dev, dt, H, G, D, E, kind, window, cap, dist, temp, rot, vmix, bs, [75, 53, 20], [1, 11, 20])


@pytest.mark.parametrize("dev,dt", OP_CASES)
@pytest.mark.parametrize("H,G,D,E,kind,window,cap,dist,temp,rot,vmix", [
    (4, 2, 64, 64, "bias", 0, 0.0, (16, 40), (0.3, 100), 0, False), (2, 1, 128, 128, "bias", 0, 0.0, (12, 70), None, 0, True),
    (4, 1, 128, 128, "cap", 150, 8.0, None, None, 32, False), (3, 1, 16, 24, "bias", 0, 0.0, (6, 100), None, 0, False)])
def test_attention_paged_long(dev, dt, H, G, D, E, kind, window, cap, dist, temp, rot, vmix):
    """Hundreds of keys: whole key tiles lie beyond the bias table's end (they take its last row as a constant) or
    outside the window, next to tiles that straddle those edges."""
    paged_case(dev, dt, H, G, D, E, kind, window, cap, dist, temp, rot, vmix, 16, [330, 290, 300], [1, 130, 300])


def paged_case(dev, dt, H, G, D, E, kind, window, cap, dist, temp, rot, vmix, bs, lens, news):
    eps, scale, lam_v = 1e-5, 0.35, 0.3
    nq, nk, nv = H * D, G * D, G * E
    ng = H * E if kind == "bias" else 0
    cols = nq + nk + nv + ng
    rows = [(torch.randn(n, cols) * 1.5).to(dt) for n in lens]
    firsts = [(torch.randn(n, nv) * 1.5).to(dt) for n in lens]
    qw, kw = 1 + 0.2 * torch.randn(D), 1 + 0.2 * torch.randn(D)
    table_rel = torch.randn(dist[0], H) * 2 if dist else None
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "scale": scale, "v_mix": vmix}
    w = {"q": selection(cols, 0, nq), "k": selection(cols, nq, nk), "v": selection(cols, nq + nk, nv),
         "q.b": torch.zeros(nq), "k.b": torch.zeros(nk), "v.b": torch.zeros(nv), "q.norm": qw, "k.norm": kw,
         "vmix": torch.tensor(lam_v), "o": torch.eye(H * E)}
    if kind == "bias":
        m.update(bias_max=dist[1], q_temp={"coef": temp[0], "every": temp[1]} if temp else None)
        w.update(rel=table_rel, g=selection(cols, nq + nk + nv, ng))
        fn = O.biased_attention
    else:
        m.update(mask={"size": window} if window else None, softcap=cap, rot={"base": 40.0, "dims": rot} if rot else None)
        fn = O.capped_window_attention
    want = torch.cat([fn(r.float(), w, m, eps, {"v_first": f.float().view(-1, G, E)} if vmix else {})[n - k:]
                      for r, f, n, k in zip(rows, firsts, lens, news)])

    table, nblk = pages(lens, bs)
    kc = torch.zeros(nblk, G, bs, D, dtype=dt, device=dev)
    vc = torch.zeros(nblk, G, E, bs, dtype=dt, device=dev)
    cs = None
    if rot:
        from vllm_distributed_amd.layers.latent_attention import interleaved_cos_sin
        cs = interleaved_cos_sin(512, rot, 40.0, torch.device(dev))
    sink = torch.zeros(H, device=dev) if kind == "bias" else None
    bias = None
    if dist:
        from vllm_distributed_amd.layers.masked_attention import log_bucket_rows
        bias = table_rel[log_bucket_rows(*dist)].contiguous().to(dev)
    mfma = ops.masked_attention_mfma_ok(H, G, D, E, 1, sink is not None, dt, dev == "cuda")
    lam = torch.tensor([lam_v], device=dev)

    def write(r, f, pos, slots):
        return ops.qk_norm_rope_cache(r.to(dev), H, G, D, E, 1, qw.to(dev), kw.to(dev), cs, pos.to(dev), rot, eps,
                                      kc, vc, slots.to(dev), by_map=mfma, pairing="neighbours", q_temp=temp,
                                      v_first=f.to(dev) if vmix else None, v_lam=lam if vmix else None)
    for s, (n, k) in enumerate(zip(lens, news)):          # context first, as earlier steps would have
        if n - k:
            pos = torch.arange(n - k)
            write(rows[s][: n - k], firsts[s][: n - k], pos, table[s, pos // bs].long() * bs + pos % bs)
    pos = torch.cat([torch.arange(n - k, n) for n, k in zip(lens, news)])
    slots = torch.cat([table[s, torch.arange(n - k, n) // bs].long() * bs + torch.arange(n - k, n) % bs
                       for s, (n, k) in enumerate(zip(lens, news))])
    new_rows = torch.cat([r[n - k:] for r, n, k in zip(rows, lens, news)])
    qn = write(new_rows, torch.cat([f[n - k:] for f, n, k in zip(firsts, lens, news)]), pos, slots)
    qsl = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32).to(dev)
    sl = torch.tensor(lens, dtype=torch.int32).to(dev)
    gt = new_rows[:, nq + nk + nv:].to(dev) if ng else None
    if mfma:
        # the matrix-core kernels: the decoded token through the decode form (whole, and with its keys dealt to three
        # workgroups), the portion and the prompt through the tiled form
        def run(splits):
            return ops.masked_softmax_attention_mfma(qn, kc, vc, table.to(dev), sl, qsl, qsl[1:] - 1, 1, 1, 2,
                                                     sum(news[1:]), 1, splits, max(news), scale, H, window, 0, sink,
                                                     1, None, eps, 1.0, gt, softcap=cap,
                                                     dist_bias=ops.padded_distance_rows(bias) if dist else None)
        got = run(1)
        assert rel(run(3), got) < 1e-2
        if D == 128:                                  # the 8-wave form for prompts, whenever the shape allows
            from vllm_distributed_amd.ops import native
            native.call("vda_set_prefill_variant", 3)
            try:
                wide = run(1)
            finally:
                native.call("vda_set_prefill_variant", 1)
            assert rel(wide, want) < OP_TOL[dt] * 3
    else:
        got = ops.masked_softmax_attention(qn, kc, vc, table.to(dev), sl, qsl, scale, window, 0, sink, 1, None, eps,
                                           1.0, gt, max(news), dt, softcap=cap, dist_bias=bias)
    assert rel(got, want) < OP_TOL[dt] * (3 if dt == torch.bfloat16 else 1)


# (heads, D, P, Dv is the latent here, latent width, window)
LATENT_SIZES = [(3, 12, 8, 24, 0), (2, 6, 12, 20, 0), (4, 16, 32, 64, 0), (4, 16, 32, 64, 19), (16, 8, 32, 128, 0),
                (5, 4, 2, 7, 6)]


@pytest.mark.parametrize("dev,dt", OP_CASES)
@pytest.mark.parametrize("H,D,P,R,window", LATENT_SIZES)
@pytest.mark.parametrize("bs", [16, 32])
def test_latent_attention_with_sinks_paged(dev, dt, H, D, P, R, window, bs):
    """Latent rows on scattered pages, a decoded token beside a portion and a whole prompt, at sizes of both kernels;
    one head's sink is large enough to take most of the weight, another's is far below every score."""
    from vllm_distributed_amd.layers.latent_attention import interleaved_cos_sin
    eps, scale = 1e-5, 0.3
    lens, news = [75, 53, 20], [1, 11, 20]
    qs = [(torch.randn(n, H * (D + P)) * 1.2).to(dt) for n in lens]
    downs = [(torch.randn(n, R + P) * 1.2).to(dt) for n in lens]
    cw = 1 + 0.2 * torch.randn(R)
    uk = torch.randn(H * D, R) / R ** 0.5
    sink = torch.randn(H)
    sink[0], sink[-1] = 16.0, -40.0

    def dense(q, down):
        """The oracle's mixer with identity projections: returns the weighted sums of the latents [L, H, R]."""
        L = q.shape[0]
        m = {"heads": H, "dim": D, "rot_dim": P, "vdim": R, "kv_rank": R, "scale": scale, "rot": {"base": 40.0}}
        c = O.unit_rms(down.float()[:, :R], eps) * cw
        k_rot = O.rotate_neighbours(down.float()[:, None, R:], P, 40.0)
        qq = q.float().view(L, H, D + P)
        q_rot = O.rotate_neighbours(qq[..., D:], P, 40.0).to(dt).float()
        c, k_rot = c.to(dt).float(), k_rot.to(dt).float()
        k = torch.cat([(c @ uk.T).view(L, H, D), k_rot.expand(L, H, P)], -1)
        v = c[:, None, :].expand(L, H, R)
        ok = O.visible(L, window or None)
        return O._attend(torch.cat([qq[..., :D], q_rot], -1), k, v, lambda d: d * m["scale"], ok, sink).view(L, H, R)
    want = torch.cat([dense(q, d)[n - k:] for q, d, n, k in zip(qs, downs, lens, news)])

    table, nblk = pages(lens, bs)
    mfma = dev == "cuda" and dt != torch.float32 and (R + P, R) in ops.MLA_KERNEL_SIZES
    kc = torch.zeros(nblk, bs, R + P, dtype=dt, device=dev)
    vt = torch.zeros(nblk, R, bs, dtype=dt, device=dev) if mfma else None
    cs = interleaved_cos_sin(128, P, 40.0, torch.device(dev))

    def write(q, down, pos, slots):
        T = q.shape[0]
        qf = torch.zeros(T, H, R + P, dtype=dt, device=dev)
        # the folded query: W_uk_h^T q_plain
        qf[:, :, :R] = torch.einsum("thd,hdr->thr", q.float().view(T, H, D + P)[..., :D],
                                    uk.view(H, D, R)).to(dt).to(dev)
        ops.latent_norm_rope_cache(q.to(dev), down.to(dev), cw.to(dev), cs, pos.to(dev), qf, kc, slots.to(dev), H, D, P,
                                   R, P, eps, vt)
        return qf
    for s, (n, k) in enumerate(zip(lens, news)):
        if n - k:
            pos = torch.arange(n - k)
            write(qs[s][: n - k], downs[s][: n - k], pos, table[s, pos // bs].long() * bs + pos % bs)
    pos = torch.cat([torch.arange(n - k, n) for n, k in zip(lens, news)])
    slots = torch.cat([table[s, torch.arange(n - k, n) // bs].long() * bs + torch.arange(n - k, n) % bs
                       for s, (n, k) in enumerate(zip(lens, news))])
    qf = write(torch.cat([q[n - k:] for q, n, k in zip(qs, lens, news)]),
               torch.cat([d[n - k:] for d, n, k in zip(downs, lens, news)]), pos, slots)
    qsl = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32).to(dev)
    sl = torch.tensor(lens, dtype=torch.int32).to(dev)
    if mfma:
        out = torch.empty(sum(news), H, R, dtype=dt, device=dev)
        for splits in (1, 3):                             # the decoded token whole and with its keys in three parts
            ops.mla_attention(out[:1], qf[:1], kc, vt, table[:1].to(dev), sl[:1], qsl[:2], scale, 1, splits,
                              window=window, sink=sink.to(dev))
            assert rel(out[:1], want[:1]) < OP_TOL[dt] * 3
        ops.mla_attention(out[1:], qf[1:], kc, vt, table[1:].to(dev), sl[1:], qsl[1:] - 1, scale, max(news), 1,
                          window=window, sink=sink.to(dev))
        got = out
    else:
        got = ops.latent_window_attention(qf, kc, table.to(dev), sl, qsl, scale, window, R, max(news), sink.to(dev))
    assert rel(got, want) < OP_TOL[dt] * (3 if dt == torch.bfloat16 else 1)
    assert want[:, 0].abs().mean() < 0.2 * want[:, -1].abs().mean()          # the large sink did take the weight


@pytest.mark.parametrize("dev", DEVICES)
def test_one_key_at_an_edge_or_far_away_decides(dev):
    """A key that carries almost all the weight: the output follows it exactly while the window lets it through -- in a
    prompt portion and for single tokens.  With a bias table whose last row is large, only the keys at least `far`
    back count, however many nearer ones there are; the extra 1 in the denominator takes the weight when every
    score is far below zero."""
    H, D, E, bs, n, needle, window = 2, 8, 4, 16, 150, 9, 6
    k_rows = 0.01 * torch.randn(n, D)
    k_rows[needle, 0] = 12.0
    v_rows = 0.01 * torch.randn(n, E)
    v_rows[needle, 0] = 5.0
    nblk = -(-n // bs)
    kc, vc = torch.zeros(nblk + 2, 1, bs, D, device=dev), torch.zeros(nblk + 2, 1, E, bs, device=dev)
    table = (torch.randperm(nblk) + 1).int().view(1, -1).to(dev)
    for p in range(n):
        kc[int(table[0, p // bs]), 0, p % bs] = k_rows[p]
        vc[int(table[0, p // bs]), 0, :, p % bs] = v_rows[p]
    q = torch.zeros(n, H, D, device=dev)
    q[:, :, 0] = 3.0

    def run(lo, hi, **kw):
        return ops.masked_softmax_attention(q[lo:hi].contiguous(), kc, vc, table,
                                            torch.tensor([hi], dtype=torch.int32, device=dev),
                                            torch.tensor([0, hi - lo], dtype=torch.int32, device=dev), 1.0,
                                            max_query_len=hi - lo, **kw).cpu().view(hi - lo, H, E)
    # the capped scores (30 at the needle, about 0 elsewhere) still single the needle out
    whole = run(0, 40, window=window, softcap=30.0)
    for p in range(40):
        seen = needle <= p < needle + window
        assert (whole[p, :, 0] > 4.9).all() == seen and (whole[p, :, 0].abs() < 0.5).all() == (not seen), p
    for p in range(needle - 1, needle + window + 2):   # single tokens and a portion that starts at the edge
        torch.testing.assert_close(run(p, p + 1, window=window, softcap=30.0)[0], whole[p])
    torch.testing.assert_close(run(needle + 3, 40, window=window, softcap=30.0), whole[needle + 3:])
    # a cap of 2 flattens the needle's score: it no longer holds all the weight among six keys
    assert (run(needle + 2, needle + 3, window=window, softcap=2.0)[0, :, 0] < 4.0).all()
    # distance bias: head 0 hears only keys at least 100 back, head 1 only those less than 3 back
    far = 100
    bias = torch.zeros(far + 1, H, device=dev)
    bias[far, 0] = 40.0
    bias[:3, 1] = 60.0
    flat = torch.zeros(n, H, D, device=dev)

    def run_flat(lo, hi):
        return ops.masked_softmax_attention(flat[lo:hi].contiguous(), kc, vc, table,
                                            torch.tensor([hi], dtype=torch.int32, device=dev),
                                            torch.tensor([0, hi - lo], dtype=torch.int32, device=dev), 1.0,
                                            max_query_len=hi - lo, dist_bias=bias).cpu().view(hi - lo, H, E)
    got = run_flat(0, n)
    for p in (needle + far - 1, needle + far, needle + far + 30):
        reach = v_rows[: p - far + 1].mean(0) if p >= far else None      # all keys at least `far` back, equally
        if p - far >= needle:
            torch.testing.assert_close(got[p, 0], reach, atol=1e-3, rtol=1e-3)
        else:
            assert got[p, 0, 0] < 0.1                                     # one short of the needle: it is not heard
        torch.testing.assert_close(got[p, 1], v_rows[p - 2: p + 1].mean(0), atol=1e-3, rtol=1e-3)
        torch.testing.assert_close(run_flat(p, p + 1)[0], got[p], atol=1e-5, rtol=1e-4)
    # every score at -20 and one more 1 in the denominator: nothing is heard; without it the mean of the values is
    low = torch.full((1, H), -20.0, device=dev)
    kw = dict(dist_bias=low)
    quiet = ops.masked_softmax_attention(flat[:30].contiguous(), kc, vc, table,
                                         torch.tensor([30], dtype=torch.int32, device=dev),
                                         torch.tensor([0, 30], dtype=torch.int32, device=dev), 1.0, max_query_len=30,
                                         sink=torch.zeros(H, device=dev), **kw).cpu().view(30, H, E)
    assert quiet.abs().max() < 1e-6
    loud = ops.masked_softmax_attention(flat[:30].contiguous(), kc, vc, table,
                                        torch.tensor([30], dtype=torch.int32, device=dev),
                                        torch.tensor([0, 30], dtype=torch.int32, device=dev), 1.0, max_query_len=30,
                                        **kw).cpu().view(30, H, E)
    torch.testing.assert_close(loud[29, 0], v_rows[:30].mean(0), atol=1e-4, rtol=1e-3)


# ---- whole models through the engine --------------------------------------------------------------------------------
VARIANTS = {
    "mixed": dict(layers=mixed_layers()),
    "latent_only": dict(layers=[O.latent_layer(mlp=None), O.latent_layer(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5,
                                                                        q_rank=2)], groups=1),
    "biased_only": dict(layers=[O.bias_layer(v_mix=True, mlp=None), O.bias_layer(q_temp=None, bias_max=6),
                                O.bias_layer(v_mix=True, heads=2, kv_heads=2, dim=6, vdim=20, q_temp=(2.0, 1))],
                        rows={0: 4, 1: 2, 2: 11}, groups=3),
    "capped_only": dict(layers=[O.cap_layer(window=1, softcap=0.5), O.cap_layer(window=None, rot_dims=12, v_mix=True),
                                O.cap_layer(softcap=None, rot_dims=0, heads=2, kv_heads=1, vdim=40, v_mix=True,
                                            mlp=None)], groups=2),
    "masks_wider_than_the_prompt": dict(layers=[O.cap_layer(window=500), O.bias_layer(bias_max=500)], rows=16),
    "odd_widths": dict(layers=[O.bias_layer(heads=3, kv_heads=1, dim=6, vdim=5, bias_max=4),
                               O.cap_layer(heads=5, kv_heads=5, dim=2, vdim=9, window=3, rot_dims=2),
                               O.latent_layer(heads=5, dim=3, rot_dim=6, vdim=7, kv_rank=11, q_rank=13)],
                       width=44, vocab=37, rows=3, groups=11),
    "experts_plain": dict(layers=[O.cap_layer(mlp=O.feed_forward(experts=5, top=1, identity=0, groups=None,
                                                                 shared=None)),
                                  O.bias_layer(mlp=O.feed_forward(experts=3, top=4, identity=1, groups=(1, 1),
                                                                  shared=8)),
                                  O.latent_layer(mlp=O.feed_forward(ff=16, experts=2, top=2, identity=4, groups=(3, 3)))],
                          width=40, vocab=50),
    "matrix_core_sizes": dict(layers=matrix_core_layers(), width=64, groups=2),
}


@pytest.mark.parametrize("dev,dtype", CASES)
@pytest.mark.parametrize("name", list(VARIANTS))
def test_whole_prompt(tmp_path, dev, dtype, name):
    kw = dict(VARIANTS[name])
    folder, cfg, W = model(tmp_path, kw.pop("layers"), seed=3, **kw)
    prompts = {"a": tokens(45, cfg["vocab"], 1), "b": tokens(1, cfg["vocab"], 2)}
    got = run_schedule(folder, dtype, dev, prompts, [[("a", 45)], [("b", 1)]], 64)
    check(cfg, W, prompts, got, dtype)


def test_residual_after_every_layer(tmp_path):
    """The framework's residual after every layer against the oracle's trail."""
    from vllm_distributed_amd.entrypoints.trace_replay import TraceReplayer
    folder, cfg, W = model(tmp_path, mixed_layers(), seed=1)
    p = tokens(12, cfg["vocab"], 1)
    _, trail = O.forward(cfg, W, p, want_layers=True)
    r = TraceReplayer(folder, "float32", 64, device="cpu", enforce_eager=True)
    seen = []
    mdl = r.core.model_executor.worker.model_runner.model
    # the residual is updated in place: a copy taken as a layer returns is the stream after that layer
    hooks = [l.register_forward_hook(lambda mod, a, out: seen.append(a[0][: len(p)].clone())) for l in mdl.layers]
    try:
        r.step([{"id": "a", "tokens": p, "want": [0]}], ["a"])
    finally:
        for h in hooks:
            h.remove()
        r.shutdown()
    assert len(seen) == len(cfg["layers"])
    torch.testing.assert_close(torch.stack(seen), trail, atol=2e-4, rtol=2e-4)


def test_a_tensor_without_a_place_is_refused(tmp_path):
    from vllm_distributed_amd.entrypoints.trace_replay import TraceReplayer
    cfg = O.make_config([O.cap_layer(mlp=None)])
    W = O.make_weights(cfg, 0)
    W["l0.mix.g"] = torch.zeros(4, 4, dtype=torch.bfloat16)              # this mixer has no output gate
    folder = O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    with pytest.raises(Exception, match="no place"):
        TraceReplayer(folder, "float32", 64, device="cpu", enforce_eager=True)


def test_benchmark_configurations_are_complete():
    """The stacks of ``bench.py --compare-lefolorn`` carry every size the model reads, the bucket count included (no
    checkpoint is there to tell it)."""
    from vllm_distributed_amd.benchmarks.hybrid_compare import SIZES, lefolorn_config
    from vllm_distributed_amd.models.lefolorn import normalise_config
    for size in SIZES.values():
        d = normalise_config(lefolorn_config(size))
        assert d["architectures"] == ["LefolornForCausalLM"] and d["num_hidden_layers"] == size["layers"]
        kinds = {l["type"] for l in d["layers"]}
        assert kinds == {"latent_attention", "attention", "attention_2"}
        assert all(l["mixer"]["bias_rows"] >= 2 for l in d["layers"] if l["type"] == "attention")
        assert d["width"] % d["norm"]["groups"] == 0


def test_tensors_the_design_never_reads_are_skipped(tmp_path):
    """A checkpoint may carry the feed-forward's scale and gate for a layer that has none, and a mixing weight for the
    layer that lends its values: they change nothing."""
    cfg = O.make_config([O.cap_layer(v_mix=True, mlp=None), O.bias_layer(v_mix=True, mlp=None)])
    W = O.make_weights(cfg, 0)
    p = tokens(9, cfg["vocab"], 1)
    want = O.forward(cfg, W, p)
    W["l0.ls2"], W["l0.rg2"], W["l0.rg2.b"] = W["l0.ls1"].clone(), W["l0.rg1"].clone(), W["l0.rg1.b"].clone()
    W["l0.mix.vmix"] = torch.tensor(0.9, dtype=torch.bfloat16)
    folder = O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    got = run_schedule(folder, "float32", "cpu", {"a": p}, [[("a", 9)]], 16)
    assert O.logit_error(got["a"], want) < TOL["float32"]


@pytest.mark.parametrize("dev,dtype", CASES)
@pytest.mark.parametrize("layers", list(LAYER_SETS))
def test_prefill_equals_decoding_token_by_token(tmp_path, dev, dtype, layers):
    folder, cfg, W = model(tmp_path, LAYER_SETS[layers](), seed=4, **({"width": 64} if layers != "mixed" else {}))
    p = tokens(70, cfg["vocab"], 5)
    sched = [[("a", 11)]] + [[("a", 1)]] * 59          # decodes 59 tokens: past windows of 9 / 21 and tables of 23 - 40
    got = run_schedule(folder, dtype, dev, {"a": p}, sched, 80)
    check(cfg, W, {"a": p}, got, dtype)
    if dev == "cpu":
        whole = run_schedule(folder, dtype, dev, {"a": p}, [[("a", 70)]], 80)
        assert O.logit_error(got["a"], whole["a"]) < 1e-4


@pytest.mark.parametrize("dev,dtype", CASES)
@pytest.mark.parametrize("block_size", [16, 32])
@pytest.mark.parametrize("layers", list(LAYER_SETS))
def test_portions_down_to_two_tokens(tmp_path, dev, dtype, block_size, layers):
    folder, cfg, W = model(tmp_path, LAYER_SETS[layers](), seed=6, **({"width": 64} if layers != "mixed" else {}))
    p = tokens(90, cfg["vocab"], 7)
    cuts = [2, 3, 11, 2, 16, 1, 17, 2, 7, 12, 1, 1, 15]
    assert sum(cuts) == 90
    got = run_schedule(folder, dtype, dev, {"a": p}, [[("a", n)] for n in cuts], 96, block_size=block_size)
    check(cfg, W, {"a": p}, got, dtype)


@pytest.mark.parametrize("dev,dtype", CASES)
@pytest.mark.parametrize("layers", list(LAYER_SETS))
def test_unequal_requests_share_steps_and_reuse_pages(tmp_path, dev, dtype, layers):
    """Seven requests, four live at most, over a pool of 10 pages: portions beside single tokens, requests that sit out
    steps, pages of finished requests taken by later ones."""
    folder, cfg, W = model(tmp_path, LAYER_SETS[layers](), seed=8, **({"width": 64} if layers != "mixed" else {}))
    V = cfg["vocab"]
    prompts = {"a": tokens(40, V, 1), "b": tokens(17, V, 2), "c": tokens(1, V, 3), "d": tokens(33, V, 4),
               "e": tokens(48, V, 5), "f": tokens(9, V, 6), "g": tokens(30, V, 7)}
    sched = [[("a", 13), ("b", 2)], [("a", 1), ("b", 15), ("c", 1)], [("a", 20), ("d", 16)],
             [("d", 1), ("a", 1)], [("a", 5), ("d", 16)],                       # a, b, c, d done: their pages return
             [("e", 31), ("f", 2)], [("e", 1), ("f", 1), ("g", 2)], [("g", 28), ("e", 1)],
             [("e", 15), ("f", 6)]]
    got = run_schedule(folder, dtype, dev, prompts, sched, 160)
    check(cfg, W, prompts, got, dtype)


NEEDLE_ROWS = 8


def reach(far):
    """The smallest distance that falls into the bias table's last row."""
    return min(n for n in range(far + 1) if O.distance_bucket(n, NEEDLE_ROWS, far) == NEEDLE_ROWS - 1)


def later_reach(far):
    """A table end a little further out whose last row starts one token later."""
    return next(f for f in range(far + 1, 2 * far) if reach(f) == reach(far) + 1)


def needle_model(window=40, far=64):
    """Token 0 is a 'needle': in the window layer one head's queries look for it and it takes nearly all the weight
    while the window lets it through; in the biased layer one head hears only the keys of the table's last row
    (``reach(far)`` tokens back and more), and the needle is much the loudest of them.  So the logits move by O(1) where
    it leaves the window and where it comes into reach of the last row."""
    layers = [O.cap_layer(heads=2, kv_heads=1, dim=8, vdim=8, window=window, rot_dims=0, scale=1.0, softcap=50.0,
                          mlp=None),
              O.bias_layer(heads=2, kv_heads=1, dim=8, vdim=8, scale=1.0, bias_max=far, q_temp=(0.1, 50), mlp=None)]
    cfg = O.make_config(layers, vocab=64, width=32, groups=1)
    W = {k: v.float() for k, v in O.make_weights(cfg, 11, rows=NEEDLE_ROWS).items()}
    emb = 0.2 * W["embed"]
    emb[:, 0] = 0
    emb[:, 2] = 3.0                                    # every token is mostly e2 ...
    emb[0] = 0
    emb[0, 0] = 6.0                                    # ... except the needle, alone along e0
    W["embed"] = emb
    for p in ("l0.", "l1."):
        q = 0.05 * W[p + "mix.q"]
        k = 0.05 * W[p + "mix.k"]
        q[0] = 0
        q[0, 2] = 4.0                                  # head 0: queries (from e2) look along direction 0
        k[0] = 0
        k[0, 0] = 4.0                                  # which only the needle (e0) fills
        W[p + "mix.q"], W[p + "mix.k"] = q, k
        W[p + "mix.q.b"], W[p + "mix.k.b"] = torch.zeros_like(W[p + "mix.q.b"]), torch.zeros_like(W[p + "mix.k.b"])
        W[p + "mix.q.norm"] = torch.full_like(W[p + "mix.q.norm"], 3.0)
        W[p + "mix.k.norm"] = torch.full_like(W[p + "mix.k.norm"], 3.0)
        W[p + "norm1"] = torch.ones_like(W[p + "norm1"])
        W[p + "rg1"] = torch.zeros_like(W[p + "rg1"])                    # gates half open everywhere
        W[p + "rg1.b"] = torch.zeros_like(W[p + "rg1.b"])
        W[p + "ls1"] = torch.ones_like(W[p + "ls1"])
    rel_ = torch.zeros_like(W["l1.mix.rel"])
    rel_[:-1, 0] = -200.0                              # head 0 of the biased layer: only the last row's keys count;
                                                       # head 1: every distance alike
    W["l1.mix.rel"] = rel_
    W["l1.mix.g"] = torch.zeros_like(W["l1.mix.g"])
    W["l1.mix.o"] = 4 * W["l1.mix.o"]                  # what the biased layer hears moves the logits visibly
    return layers, cfg, {k: v.to(torch.bfloat16) for k, v in W.items()}


@pytest.mark.parametrize("dev,dtype", CASES)
def test_far_key_and_edges_that_matter(tmp_path, dev, dtype):
    layers, cfg, W = needle_model()
    folder = O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    V = cfg["vocab"]
    body = [t % (V - 1) + 1 for t in tokens(400, V, 12)]
    assert reach(64) == 32
    prompts = {"first": [0] + body[:150],                     # needle at the very first position
               "edge": [0] + body[:120],                      # reached by the last row at 32, leaves the window at 40
               "late": body[:30] + [0] + body[30:100],        # reached at 62, leaves at 70, both as single tokens
               "far": body[:50] + [0] + body[50:330]}         # far back, over many pages
    sched = [[("first", 100), ("edge", 30)], [("first", 1), ("edge", 1)], [("first", 50), ("edge", 10)],
             [("edge", 1), ("late", 62)]] + [[("edge", 1), ("late", 1)]] * 3 + [[("late", 1)]] * 7 + \
            [[("edge", 76), ("far", 200), ("late", 1)], [("far", 129), ("late", 28)], [("far", 1)], [("far", 1)]]
    got = run_schedule(folder, dtype, dev, prompts, sched, 640)
    check(cfg, W, prompts, got, dtype)
    # the crafted edges are real: a window one token shorter, or a table that reaches one token later, changes the
    # logits exactly there
    full = {rid: O.forward(cfg, W, prompts[rid]) for rid in ("edge", "late")}
    # (nothing precedes the needle of "edge", so before the last row reaches it that row is empty either way)
    for which, key, value, rid, pos in ((0, "mask", {"size": 39}, "edge", 39), (0, "mask", {"size": 39}, "late", 69),
                                        (1, "bias_max", later_reach(64), "edge", 32)):
        ls = [dict(l, mixer=dict(l["mixer"])) for l in layers]
        ls[which]["mixer"][key] = value
        other = O.forward(O.make_config(ls, vocab=64, width=32, groups=1), W, prompts[rid])
        assert O.logit_error(other[pos], full[rid][pos]) > 0.01 > O.logit_error(other[pos - 1], full[rid][pos - 1]), \
            (which, rid)


@pytest.mark.parametrize("dev,dtype", CASES)
def test_far_key_among_hundreds(tmp_path, dev, dtype):
    """A window of 300 and a table whose last row starts 296 back: the one key that matters sits hundreds of tokens and
    many pages back, comes into the last row's reach and leaves the window while single tokens are decoded."""
    far = next(f for f in range(300, 3000) if reach(f) == 296)
    layers, cfg, W = needle_model(window=300, far=far)
    folder = O.save_checkpoint(str(tmp_path / "m"), cfg, W)
    V = cfg["vocab"]
    body = [t % (V - 1) + 1 for t in tokens(400, V, 14)]
    p = [0] + body[:345]                                   # needle at 0: in reach from 296, in the window up to 299
    sched = [[("deep", 290)]] + [[("deep", 1)]] * 22 + [[("deep", 2)], [("deep", 3)], [("deep", 29)]]
    got = run_schedule(folder, dtype, dev, {"deep": p}, sched, 384)
    check(cfg, W, {"deep": p}, got, dtype)
    full = O.forward(cfg, W, p)
    for which, key, value, pos in ((0, "mask", {"size": 299}, 299), (1, "bias_max", later_reach(far), 296)):
        ls = [dict(l, mixer=dict(l["mixer"])) for l in layers]
        ls[which]["mixer"][key] = value
        other = O.forward(O.make_config(ls, vocab=64, width=32, groups=1), W, p)
        assert O.logit_error(other[pos], full[pos]) > 0.01 > O.logit_error(other[pos - 1], full[pos - 1]), which


@pytest.mark.parametrize("dev", DEVICES)
def test_greedy_generation_through_llm(tmp_path, dev):
    """The engine's own entry point and scheduler: greedy continuation of three prompts of unequal length equals
    the oracle's (recomputed from scratch for every token)."""
    from vllm_distributed_amd import LLM, SamplingParams
    folder, cfg, W = model(tmp_path, mixed_layers(), seed=9)
    V = cfg["vocab"]
    prompts = [tokens(19, V, 1), tokens(3, V, 2), tokens(33, V, 3)]
    llm = LLM(model=folder, skip_tokenizer_init=True, dtype="float32", device=dev, max_model_len=128, max_num_seqs=4,
              max_num_batched_tokens=24, enable_chunked_prefill=True, gpu_memory_utilization=0.1, enforce_eager=True)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(temperature=0, max_tokens=10,
                                                                                 ignore_eos=True))
    llm.shutdown()
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.outputs[0].token_ids:
            logits = O.forward(cfg, W, seq)[-1]
            best = int(logits.argmax())
            assert tok == best or logits[best] - logits[tok] < 1e-3, (len(seq), tok, best)
            seq.append(tok)
        assert len(o.outputs[0].token_ids) == 10


def test_long_decoding(tmp_path):
    """300 single tokens after a short prompt: nothing drifts against the oracle's whole-sequence run."""
    folder, cfg, W = model(tmp_path, mixed_layers()[:3], seed=12)
    p = tokens(305, cfg["vocab"], 13)
    got = run_schedule(folder, "float32", "cpu", {"a": p}, [[("a", 5)]] + [[("a", 1)]] * 300, 320)
    check(cfg, W, {"a": p}, got, "float32")


@pytest.mark.gpu
@pytest.mark.parametrize("layers", list(LAYER_SETS))
def test_decode_graphs_equal_eager(tmp_path, layers):
    """Single decoded tokens through captured graphs (several replays with other work between them) give the
    eager logits."""
    folder, cfg, W = model(tmp_path, LAYER_SETS[layers](), seed=10, **({"width": 64} if layers != "mixed" else {}))
    V = cfg["vocab"]
    prompts = {"a": tokens(30, V, 1), "b": tokens(22, V, 2)}
    sched = [[("a", 10), ("b", 4)]] + [[("a", 1), ("b", 1)]] * 18 + [[("a", 2)]]
    eager = run_schedule(folder, "bfloat16", "cuda", prompts, sched, 64, eager=True)
    graph = run_schedule(folder, "bfloat16", "cuda", prompts, sched, 64, eager=False)
    for k in prompts:
        torch.testing.assert_close(graph[k], eager[k], atol=1e-3, rtol=1e-3)
