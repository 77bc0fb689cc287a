"""Kepusun family against the plain oracle (tests/kepusun_oracle.py).

Every test builds its own small configuration and random checkpoint,
loads it through the framework's registry and loader, and drives the
framework's stage, cache and batcher. The same bodies run on the CPU tier
(torch ops) and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""

import json
import math
import os

import pytest
import torch

import kepusun_oracle as O
from tensorlink_amd.engine.batcher import ContinuousBatcher
from tensorlink_amd.models.paged import PAGE, HybridSlotCache
from tensorlink_amd.ops import mixers as mx
from tensorlink_amd.parallel.pipeline import PipelineRunner, SamplingParams
from tensorlink_amd.parallel.planner import plan_for_world

CPU32 = pytest.param("cpu", torch.float32, id="cpu-f32")
GPU32 = pytest.param("cuda", torch.float32, id="gpu-f32",
                     marks=pytest.mark.gpu)
GPU16 = pytest.param("cuda", torch.bfloat16, id="gpu-bf16",
                     marks=pytest.mark.gpu)
ALL = [CPU32, GPU32, GPU16]


def tol(dtype):
    return 5e-4 if dtype == torch.float32 else 6e-2


# ------------------------------------------------------------ fixtures
def moe(experts, top, count, keep, ff, scale):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "scale": scale,
                       "groups": {"count": count, "keep": keep}}}


def att(heads, kv, dim, vdim, scale, diff, kv_from=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
         "scale": scale, "diff": diff}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def cfg_mixed():
    """Attention first, shared KV later, a layer without feed-forward,
    three streams, vdim != dim, grouped-GEMM-friendly expert sizes."""
    return {"architecture": "Kepusun", "vocab": 96, "width": 64,
            "streams": 3, "norm": {"eps": 1e-5}, "layers": [
                {"type": "attention", "mixer": att(4, 2, 16, 24, 0.3, 0.35),
                 "mlp": moe(8, 2, 4, 2, 64, 1.5)},
                {"type": "mlstm", "mixer": {"heads": 2, "dim": 24,
                                            "vdim": 40, "gate_cap": 8.0},
                 "mlp": None},
                {"type": "attention",
                 "mixer": att(4, 2, 16, 24, 0.3, 0.2, kv_from=0),
                 "mlp": moe(6, 3, 3, 3, 40, 1.0)},
                {"type": "mlstm", "mixer": {"heads": 3, "dim": 8,
                                            "vdim": 72, "gate_cap": 20.0},
                 "mlp": moe(8, 2, 4, 2, 64, 1.5)}]}


def cfg_ones():
    """Values that could hide a fault by being equal or 1: one stream, one
    group, top 1, kv_heads == heads, one head."""
    return {"architecture": "Kepusun", "vocab": 50, "width": 32,
            "streams": 1, "norm": {"eps": 1e-6}, "layers": [
                {"type": "mlstm", "mixer": {"heads": 1, "dim": 16,
                                            "vdim": 16, "gate_cap": 12.0},
                 "mlp": moe(4, 1, 1, 1, 24, 2.5)},
                {"type": "attention", "mixer": att(2, 2, 12, 12, 0.25, 0.5),
                 "mlp": moe(4, 1, 1, 1, 24, 2.5)}]}


def cfg_tiles():
    """Head sizes the MFMA prompt kernel serves in bf16 (dim % 8 == 0,
    vdim % 16 == 0), one with a padded 32-wide d-chunk."""
    return {"architecture": "Kepusun", "vocab": 80, "width": 64,
            "streams": 2, "norm": {"eps": 1e-6}, "layers": [
                {"type": "attention", "mixer": att(4, 2, 24, 48, 0.2, 0.4),
                 "mlp": moe(4, 2, 2, 1, 64, 1.0)},
                {"type": "mlstm", "mixer": {"heads": 2, "dim": 32,
                                            "vdim": 64, "gate_cap": 10.0},
                 "mlp": None},
                {"type": "attention",
                 "mixer": att(4, 2, 24, 48, 0.2, 0.6, kv_from=0),
                 "mlp": None}]}


def make_weights(cfg, seed=0):
    """Random checkpoint tensors (bf16-representable fp32), named as in a
    checkpoint file."""
    g = torch.Generator().manual_seed(seed)
    w, ns = cfg["width"], cfg["streams"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    P = {"embed": rnd(cfg["vocab"], w), "head": rnd(cfg["vocab"], w,
                                                   std=w ** -0.5)}

    def norm(name):
        P[name] = 1.0 + rnd(w, std=0.1)
        P[name + ".b"] = rnd(w, std=0.1)
        P[name + ".alpha"] = (0.6 + rnd(1, std=0.1)).reshape(())

    def hc(name):
        P[name + ".in"] = (torch.full((ns,), 1.0 / ns) + rnd(ns, std=0.1)
                           ).bfloat16().float()
        P[name + ".out"] = (1.0 + rnd(ns, std=0.1)).bfloat16().float()
        P[name + ".mix"] = (torch.eye(ns) + rnd(ns, ns, std=0.1)
                            ).bfloat16().float()

    norm("final.norm")
    for i, lc in enumerate(cfg["layers"]):
        a, mc = f"l{i}.", lc["mixer"]
        norm(a + "norm1")
        hc(a + "hc1")
        H, D, V = mc["heads"], mc["dim"], mc["vdim"]
        s = w ** -0.5
        if lc["type"] == "mlstm":
            for nm, rows in (("q", H * D), ("k", H * D), ("v", H * V),
                             ("g", H * V)):
                P[a + "mix." + nm] = rnd(rows, w, std=2 * s)
            P[a + "mix.o"] = rnd(w, H * V, std=(H * V) ** -0.5)
            P[a + "mix.norm"] = 1.0 + rnd(H * V, std=0.1)
            for nm in "if":
                P[a + f"mix.{nm}"] = rnd(H, w, std=3 * s)
                P[a + f"mix.{nm}.b"] = rnd(H, std=2.0)
        else:
            G = mc["kv_heads"]
            P[a + "mix.q"] = rnd(H * 2 * D, w, std=2 * s)
            if "kv_from" not in mc:
                P[a + "mix.k"] = rnd(G * 2 * D, w, std=2 * s)
                P[a + "mix.v"] = rnd(G * V, w, std=2 * s)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                P[a + "mix." + nm] = rnd(D, std=0.3)
            P[a + "mix.o"] = rnd(w, H * V, std=(H * V) ** -0.5)
        if lc.get("mlp") is not None:
            norm(a + "norm2")
            hc(a + "hc2")
            E, ff = lc["mlp"]["router"]["experts"], lc["mlp"]["expert"]["ff"]
            P[a + "mlp.router"] = rnd(E, w, std=4 * s)
            for e in range(E):
                P[a + f"mlp.e{e}.up"] = rnd(ff, w, std=2 * s)
                P[a + f"mlp.e{e}.down"] = rnd(w, ff, std=ff ** -0.5)
    # exactly what a bf16 checkpoint holds
    return {k: v.bfloat16().float() for k, v in P.items()}


def write_checkpoint(path, cfg, P):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in P.items()},
              os.path.join(path, "model.safetensors"))


_CACHE = {}


def model(tmp_path_factory, cfg_fn, device, dtype, seed=0):
    """(runner, oracle weights, cfg) — checkpoint written once per
    configuration, loaded through the registry by directory name."""
    key = (cfg_fn.__name__, seed)
    if key not in _CACHE:
        cfg = cfg_fn()
        P = make_weights(cfg, seed)
        d = str(tmp_path_factory.mktemp(cfg_fn.__name__))
        write_checkpoint(d, cfg, P)
        _CACHE[key] = (d, cfg, P)
    d, cfg, P = _CACHE[key]
    plan = plan_for_world(d, 1)
    runner = PipelineRunner(plan, 0, 1, device=torch.device(device),
                            init="checkpoint", ckpt_dir=d, dtype=dtype)
    return runner, P, cfg


def batcher(runner, max_ctx=512, pool_pages=None, slots=4):
    return ContinuousBatcher(runner, max_slots=slots, max_ctx=max_ctx,
                             pool_pages=pool_pages)


def oracle(toks, P, cfg, **kw):
    """The plain oracle in float64: some positions of a random model are
    ill-conditioned (a1 - lambda a2 nearly cancels before its unit norm),
    where an fp32 oracle is itself off by more than the product."""
    torch.set_default_dtype(torch.float64)
    try:
        return O.forward(toks, {k: v.double() for k, v in P.items()}, cfg,
                         **kw)
    finally:
        torch.set_default_dtype(torch.float32)


def rel_err(got, want):
    got, want = got.float().cpu(), want.float().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-6)


def close(got, want, dtype):
    """fp32: every position within tolerance of the exact oracle.

    bf16 results are compared with the framework's own whole-prompt bf16
    logits (see ``reference``): a random model is chaotic under bf16
    rounding (a near-tie of the router flips, a cancelling a1 - lambda a2
    is amplified, and the recurrent state carries the difference on), so
    only the bulk of the positions is held tight there; exactness is the
    fp32 runs' job."""
    e = rel_err(got, want).reshape(-1)
    if dtype == torch.float32:
        ok = float(e.max()) < tol(dtype)
    else:
        ok = (float(e.median()) < tol(dtype) / 2
              and float((e > 3 * tol(dtype)).float().mean()) <= 0.1)
    if not ok:
        print("rel err: median %.3g max %.3g" % (float(e.median()),
                                                 float(e.max())))
    return ok


def reference(runner, toks, P, cfg, dtype):
    """What a schedule's logits are compared with: the exact oracle in
    fp32; in bf16 the same request alone, whole, through the framework
    (itself checked against the oracle in the bulk)."""
    want = oracle(toks, P, cfg)
    if dtype == torch.float32:
        return want
    own = run_schedule(batcher(runner, max_ctx=max(512, len(toks))), toks,
                       [len(toks)], rid="ref")
    assert float(rel_err(own, want).median()) < tol(dtype)
    return own


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def run_schedule(b, toks, cuts, rid="r"):
    """Feed ``toks`` in portions of the given sizes (rest one by one);
    returns logits at every position."""
    outs, at = [], 0
    sizes = list(cuts)
    while at < len(toks):
        n = sizes.pop(0) if sizes else 1
        n = min(n, len(toks) - at)
        last = at + n == len(toks)
        outs.append(b.forced_step([(rid, toks[at:at + n], list(range(n)))],
                                  [rid] if last else []))
        at += n
    return torch.cat(outs)


# ------------------------------------------------- mechanisms, one by one
@pytest.mark.parametrize("device,dtype", ALL)
def test_hyper_dyt_op(device, dtype):
    g = torch.Generator().manual_seed(1)
    for ns in (1, 2, 3, 5):
        T, W = 7, 24
        X = torch.randn(ns, T, W, generator=g)
        y = torch.randn(T, W, generator=g).to(dtype)
        mix = torch.randn(ns, ns, generator=g)
        out = torch.randn(ns, generator=g)
        inw = torch.randn(ns, generator=g)
        al = torch.tensor([0.7])
        w, b = torch.randn(W, generator=g), torch.randn(W, generator=g)
        Xn = [sum(mix[s, t] * X[s] for s in range(ns)) + out[t] * y.float()
              for t in range(ns)]
        u = sum(inw[s] * Xn[s] for s in range(ns))
        want = torch.tanh(al * u) * w + b
        Xd = X.clone().to(device)
        h, us = mx.hyper_dyt(Xd, y.to(device), mix.to(device),
                             out.to(device), inw.to(device), al.to(device),
                             w.to(device), b.to(device), out_dtype=dtype,
                             want_sum=True)
        assert torch.allclose(Xd.cpu(), torch.stack(Xn), atol=1e-5)
        assert torch.allclose(us.cpu(), u, atol=1e-5)
        assert torch.allclose(h.float().cpu(), want,
                              atol=1e-5 if dtype == torch.float32 else 2e-2)
        # read-only form: plain sum of the streams, no norm
        _, s2 = mx.hyper_dyt(Xd, want_sum=True)
        assert torch.allclose(s2.cpu(), torch.stack(Xn).sum(0), atol=1e-5)


def test_router_groups_against_oracle():
    g = torch.Generator().manual_seed(2)
    for E, top, cnt, keep in ((12, 3, 4, 2), (8, 1, 1, 1), (6, 6, 3, 3),
                              (16, 2, 8, 1)):
        W = 20
        P = {"r.router": torch.randn(E, W, generator=g)}
        h = torch.randn(9, W, generator=g)
        rc = {"experts": E, "top": top, "scale": 1.7,
              "groups": {"count": cnt, "keep": keep}}
        chosen, weights = O.moe_route(h, P, "r.", rc)
        w, idx = mx.group_limited_router(h @ P["r.router"].T, top, cnt,
                                         keep, 1.7)
        for t in range(9):
            got = dict(zip(idx[t].tolist(), w[t].tolist()))
            assert sorted(got) == sorted(chosen[t])
            for e, ww in zip(chosen[t], weights[t]):
                assert abs(got[e] - float(ww)) < 1e-6
        if keep < cnt:
            per = E // cnt
            assert all(len({e // per for e in c}) <= keep for c in chosen)


def _one_seq_meta(cache, n, pos0, device, slot=0):
    cache.ensure(slot, pos0 + n)
    return mx.RaggedMeta([n], [pos0], [slot], cache.table[[slot]], device)


@pytest.mark.parametrize("T,hdv", [(37, (3, 20, 28)), (333, (3, 20, 28)),
                                   (37, (2, 72, 40)), (333, (1, 136, 24)),
                                   (300, (1, 16, 272)), (37, (2, 48, 64))],
                         ids=lambda x: str(x).replace(" ", ""))
@pytest.mark.parametrize("device,dtype", ALL)
def test_mlstm_mixer_against_oracle(device, dtype, T, hdv):
    """The mixer alone, whole sequence and token by token through the
    state slot; biases push some tokens onto each branch of the
    normaliser max(|n.q|, exp(-m)). The long sequence takes the
    chunk-parallel form on the GPU (summaries, chain, read-out), also as a
    continuation of a state left by an earlier portion."""
    from tensorlink_amd.models.mixers import MLSTMMixer
    g = torch.Generator().manual_seed(3)
    (H, D, V), W, cap, eps = hdv, 48, 6.0, 1e-5   # every register tiling
    r = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std
                             ).bfloat16().float()
    P = {"m.q": r(H * D, W, std=.3), "m.k": r(H * D, W, std=.3),
         "m.v": r(H * V, W, std=.3), "m.g": r(H * V, W, std=.3),
         "m.o": r(W, H * V, std=.1), "m.norm": 1 + r(H * V, std=.1),
         "m.i": r(H, W, std=.5), "m.f": r(H, W, std=.5),
         "m.i.b": torch.tensor([-6.0, 0.0, 4.0])[:H],
         "m.f.b": torch.tensor([3.0, -1.0, 0.5])[:H]}
    h = r(T, W)
    mc = {"heads": H, "dim": D, "vdim": V, "gate_cap": cap}
    want = O.mlstm_sequence(h, P, "m.", mc, eps)
    mod = MLSTMMixer(W, H, D, V, cap, eps)
    with torch.no_grad():
        mod.proj.weight.copy_(torch.cat([P["m.q"], P["m.k"], P["m.v"],
                                         P["m.g"]]))
        mod.gate.weight.copy_(torch.cat([P["m.i"], P["m.f"]]))
        mod.gate.bias.copy_(torch.cat([P["m.i.b"], P["m.f.b"]]))
        mod.norm.copy_(P["m.norm"])
        mod.o_proj.weight.copy_(P["m.o"])
    mod.to(device=device, dtype=dtype)
    cache = HybridSlotCache([mod.cache_spec()], 4, 12, 512, device, dtype)
    hd = h.to(device=device, dtype=dtype)
    cut = 11 if T < 100 else 40         # second portion of 293 tokens
    with torch.no_grad():
        whole = mod(hd, _one_seq_meta(cache, T, 0, device, slot=1), cache, 0)
        steps = [mod(hd[t:t + 1], _one_seq_meta(cache, 1, t, device, slot=2),
                     cache, 0) for t in range(T)]
        parts = [mod(hd[:cut], _one_seq_meta(cache, cut, 0, device, slot=3),
                     cache, 0),
                 mod(hd[cut:], _one_seq_meta(cache, T - cut, cut, device,
                                             slot=3), cache, 0)]
    scale = float(want.abs().max())
    for got in (whole, torch.cat(steps), torch.cat(parts)):
        err = (got.float().cpu() - want).abs()
        if dtype == torch.float32:
            assert float(err.max()) < 2e-5 * scale
        else:
            # bf16 q/k/v rounding accumulates in the state over hundreds
            # of tokens: tight in the bulk, bounded at the worst element
            assert float(err.median()) < 1e-2 * scale
            assert float(err.max()) < 0.3 * scale
    if dtype != torch.float32:
        # ... and the three schedules agree with each other tightly
        for got in (torch.cat(steps), torch.cat(parts)):
            d = (got.float() - whole.float()).abs().cpu()
            assert float(d.max()) < 3e-2 * scale
    # the slot state after the whole / cut / stepped runs agrees
    for a, b_ in zip(cache.state[0], cache.state[0]):
        for s2 in (2, 3):
            assert torch.allclose(a[1].cpu(), b_[s2].cpu(), rtol=1e-3,
                                  atol=1e-4 * float(a[1].abs().max()))


@pytest.mark.parametrize("dims", [(4, 2, 8, 12), (4, 2, 16, 32),
                                  (2, 1, 40, 80), (3, 3, 72, 16),
                                  (2, 1, 16, 160), (1, 1, 12, 300)],
                         ids=lambda d: "H%dG%dD%dV%d" % d)
@pytest.mark.parametrize("device,dtype", ALL)
def test_diff_attention_far_key_and_page_edges(device, dtype, dims):
    """The op alone on crafted rows: for each query one key far back gets a
    dominant score in map 1 and another in map 2, so a lost key, an
    off-by-one causal edge or a wrong page shows; queries sit just before,
    on and after page borders, in a prompt portion and decoded alone."""
    H, G, D, V = dims       # some serve the MFMA tile kernel in bf16
    L = 5 * PAGE + 9        # decoding past 512 keys: split-key rows merge
    g = torch.Generator().manual_seed(4)
    k = torch.randn(L, G, 2, D, generator=g) * 0.1
    v = torch.randn(L, G, V, generator=g)
    q = torch.randn(L, H, 2, D, generator=g) * 0.1
    probes = [0, 1, 2, PAGE - 1, PAGE, PAGE + 1, 2 * PAGE - 1, 2 * PAGE,
              4 * PAGE - 1, 4 * PAGE, 4 * PAGE + 1, 5 * PAGE, L - 1]
    for t in probes:
        # the query's own position and position 0 carry the two big keys:
        # exactly the keys an exclusive edge or a dropped first page loses
        for hh in range(H):
            q[t, hh, 0] = 0.0
            q[t, hh, 0, hh % D] = 6.0
            q[t, hh, 1] = 0.0
            q[t, hh, 1, (hh + 1) % D] = 6.0
    for gg in range(G):
        for t in probes:
            k[t, gg, 0, :4] = 6.0 * (t + 1) / L
        k[0, gg, 1, :] = 5.0
    scale, diff, eps, lam = 0.7, 0.3, 1e-6, torch.tensor([0.55])
    k, v, q = (x.bfloat16().float() for x in (k, v, q))

    def plain(t):
        out = torch.zeros(H, V)
        for hh in range(H):
            gi = hh // (H // G)
            a = [torch.softmax((k[:t + 1, gi, mp] @ q[t, hh, mp]) * scale, 0)
                 @ v[:t + 1, gi] for mp in range(2)]
            out[hh] = O.unit_rms(a[0] - lam * a[1], eps) * (1 - diff)
        return out.reshape(-1)

    want = torch.stack([plain(t) for t in range(L)])
    spec = {"kind": "kv", "G": G, "DK": 2 * D, "V": V}
    cache = HybridSlotCache([spec], 2, 8, 1024, device, dtype)
    # pages leased out of order: the table is a real indirection
    cache.ensure(1, PAGE)
    cache.ensure(0, L)
    cache.release_slot(1)
    rows = torch.cat([q.reshape(L, -1), k.reshape(L, -1),
                      v.reshape(L, -1)], 1).to(device=device, dtype=dtype)
    qc, kc = H * 2 * D, G * 2 * D
    cut = PAGE + 1                     # prompt portion, then one by one
    got = []
    for lo, hi in [(0, cut)] + [(t, t + 1) for t in range(cut, L)]:
        meta = mx.RaggedMeta([hi - lo], [lo], [0], cache.table[[0]], device)
        mx.kv_append(rows[lo:hi], qc, qc + kc, cache.k[0], cache.v[0], meta)
        got.append(mx.diff_attention(rows[lo:hi], 0, cache.k[0], cache.v[0],
                                     meta, lam.to(device), H, D, scale, diff,
                                     eps))
    got = torch.cat(got).float().cpu()
    t_ = 2e-5 if dtype == torch.float32 else 3e-2
    assert float((got - want).abs().max()) < t_ * float(want.abs().max())


# --------------------------------------------------- whole model, engine
@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("cfg_fn", [cfg_mixed, cfg_ones, cfg_tiles])
def test_whole_prompt_matches_oracle(tmp_path_factory, cfg_fn, device,
                                     dtype):
    runner, P, cfg = model(tmp_path_factory, cfg_fn, device, dtype)
    toks = tokens(cfg, PAGE + 30, 5)
    want, layers = oracle(toks, P, cfg, return_layers=True)
    b = batcher(runner)
    got = run_schedule(b, toks, [len(toks)])
    if dtype == torch.float32:
        assert close(got, want, dtype)
    else:
        assert float(rel_err(got, want).median()) < tol(dtype)
    # the residual after every layer, through the stage's own hook
    stage = runner.stage
    stage.layer_sums = []
    try:
        run_schedule(batcher(runner), toks, [len(toks)])
        for u, w in zip(stage.layer_sums, layers):
            if dtype == torch.float32:
                assert close(u, w, dtype)
            else:
                assert float(rel_err(u, w).median()) < tol(dtype)
    finally:
        stage.layer_sums = None


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("cfg_fn", [cfg_mixed, cfg_tiles])
def test_portions_and_decode_match_whole(tmp_path_factory, cfg_fn, device,
                                         dtype):
    """Prefill against token-by-token decoding and portions of several
    sizes (down to two tokens, across a page border)."""
    runner, P, cfg = model(tmp_path_factory, cfg_fn, device, dtype)
    toks = tokens(cfg, PAGE + 21, 6)
    want = reference(runner, toks, P, cfg, dtype)
    for cuts in ([1] * 0, [PAGE - 1, 2, 2, 5], [2, 3, 64, 61, 7],
                 [len(toks) - 12]):
        got = run_schedule(batcher(runner), toks, cuts)
        assert close(got, want, dtype), cuts


@pytest.mark.parametrize("device,dtype", ALL)
def test_mixed_batch_and_reuse_of_slots_and_pages(tmp_path_factory, device,
                                                  dtype):
    """Unequal requests in one batch equal each alone; the pool is so
    small that pages and slots of finished requests are used again by
    requests of other lengths."""
    runner, P, cfg = model(tmp_path_factory, cfg_tiles, device, dtype)
    lens = {"a": 150, "b": 40, "c": 9, "d": 131, "e": 70, "f": 3}
    toks = {r: tokens(cfg, n, 10 + i) for i, (r, n) in
            enumerate(lens.items())}
    want = {r: reference(runner, t, P, cfg, dtype) for r, t in toks.items()}
    b = batcher(runner, max_ctx=256, pool_pages=5, slots=3)
    got = {r: [] for r in toks}
    at = {r: 0 for r in toks}
    # (request, tokens this step) per step; d, e, f reuse a, b, c's slots
    plan = [[("a", 100), ("b", 7)], [("a", 2), ("b", 1), ("c", 9)],
            [("a", 48), ("b", 32)], [("d", 3)], [("d", 128), ("e", 1)],
            [("e", 69), ("f", 2)], [("f", 1)]]
    used_slots = []
    for step in plan:
        entries, ends = [], []
        for r, n in step:
            entries.append((r, toks[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == lens[r]:
                ends.append(r)
        used_slots += [b._forced.get(r) for r, _ in step]
        out = b.forced_step(entries, ends)
        o = 0
        for r, n in step:
            got[r].append(out[o:o + n])
            o += n
    assert b.cache.available_pages() == 5 and not b._forced
    for r in toks:
        assert at[r] == lens[r]
        assert close(torch.cat(got[r]), want[r], dtype), r


@pytest.mark.parametrize("device,dtype", ALL)
def test_long_prompts_in_one_batch(tmp_path_factory, device, dtype):
    """Prompts long enough for the chunk-parallel recurrence and several
    attention tiles, two of unequal length in one step, the longer one
    continued by a second long portion."""
    runner, P, cfg = model(tmp_path_factory, cfg_tiles, device, dtype)
    ta, tb = tokens(cfg, 610, 31), tokens(cfg, 77, 32)
    wa = reference(runner, ta, P, cfg, dtype)
    wb = reference(runner, tb, P, cfg, dtype)
    b = batcher(runner, max_ctx=1024)
    o1 = b.forced_step([("a", ta[:300], list(range(300))),
                        ("b", tb, list(range(77)))], ["b"])
    o2 = b.forced_step([("a", ta[300:], list(range(310)))], ["a"])
    assert close(torch.cat([o1[:300], o2]), wa, dtype)
    assert close(o1[300:], wb, dtype)


@pytest.mark.parametrize("device,dtype", [CPU32, GPU32])
def test_long_decode(tmp_path_factory, device, dtype):
    runner, P, cfg = model(tmp_path_factory, cfg_ones, device, dtype)
    toks = tokens(cfg, 2 * PAGE + 40, 7)
    want = oracle(toks, P, cfg)
    got = run_schedule(batcher(runner), toks, [5])
    assert close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", [CPU32, GPU32])
def test_greedy_generation_through_scheduler(tmp_path_factory, device,
                                             dtype):
    """submit() -> scheduler thread -> sampled tokens, two requests of
    unequal length concurrently with portioned prefill; each must equal
    greedy decoding with the oracle. Also PipelineRunner.generate."""
    runner, P, cfg = model(tmp_path_factory, cfg_mixed, device, dtype)
    prompts = [tokens(cfg, 19, 21), tokens(cfg, 6, 22)]
    new = 6

    def greedy(p):
        seq = list(p)
        for _ in range(new):
            seq.append(int(oracle(seq, P, cfg)[-1].argmax()))
        return seq[len(p):]

    want = [greedy(p) for p in prompts]
    b = ContinuousBatcher(runner, max_slots=2, max_ctx=128,
                          prefill_chunk=8).start()
    try:
        reqs = [b.submit(torch.tensor(p), max_new_tokens=new)
                for p in prompts]
        outs = [r.result() for r in reqs]
    finally:
        b.stop()
    assert outs == want
    out = runner.generate(torch.tensor([prompts[0]]),
                          SamplingParams(max_new_tokens=new))
    assert out[0].tolist() == want[0]


def test_config_and_loader_are_strict(tmp_path):
    cfg = cfg_ones()
    P = make_weights(cfg)
    d = str(tmp_path / "m")
    write_checkpoint(d, cfg, P)
    from tensorlink_amd.models.configs import get_config
    c = get_config(d)
    assert c.architecture == "kepusun" and c.streams == 1
    assert c.param_count() == sum(v.numel() for v in P.values())
    rt = type(c).from_json(c.to_json())
    assert rt.layer_specs == c.layer_specs
    bad = dict(P)
    bad.pop("l1.mix.lq2")
    d2 = str(tmp_path / "bad")
    write_checkpoint(d2, cfg, bad)
    with pytest.raises(KeyError):
        PipelineRunner(plan_for_world(d2, 1), 0, 1,
                       device=torch.device("cpu"), init="checkpoint",
                       ckpt_dir=d2, dtype=torch.float32)
    cfg2 = cfg_ones()
    cfg2["layers"][1]["mixer"]["kv_from"] = 0      # not an attention layer
    d3 = str(tmp_path / "bad2")
    write_checkpoint(d3, cfg2, P)
    with pytest.raises(KeyError):
        get_config(d3)


def test_single_stream_without_hyper_connection_tensors(tmp_path):
    """One stream and no hc tensors in the checkpoint is the plain
    pre-norm residual x + f(norm(x))."""
    cfg = cfg_ones()
    P = make_weights(cfg, seed=3)
    for k in list(P):
        if ".hc" in k:
            P[k] = torch.ones_like(P[k])
    d = str(tmp_path / "m")
    write_checkpoint(d, cfg, {k: v for k, v in P.items() if ".hc" not in k})
    runner = PipelineRunner(plan_for_world(d, 1), 0, 1,
                            device=torch.device("cpu"), init="checkpoint",
                            ckpt_dir=d, dtype=torch.float32)
    toks = tokens(cfg, 40, 9)
    got = run_schedule(batcher(runner), toks, [17, 2])
    assert close(got, oracle(toks, P, cfg), torch.float32)
