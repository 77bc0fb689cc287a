"""Plain, slow fp32 oracle for the Kepusun design, one function per
mechanism, written token by token from the equations. It shares no code
with the serving path: every loop is explicit and nothing is batched,
chunked, cached or paged.

Notation: ``P`` is a dict name -> float32 tensor, ``cfg`` the parsed
configuration dict (same keys as a checkpoint's ``config.json``).
"""

from __future__ import annotations

import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyt(x, P, name):
    """Dynamic Tanh: tanh(alpha x) * w + b — no statistics."""
    return torch.tanh(P[name + ".alpha"] * x) * P[name] + P[name + ".b"]


# ------------------------------------------------------------------ mixers
def mlstm_sequence(h, P, pre, mc, eps):
    """Matrix-memory recurrence over one whole sequence h [T, W]."""
    H, D, V, cap = mc["heads"], mc["dim"], mc["vdim"], mc["gate_cap"]
    T = h.shape[0]
    q = (h @ P[pre + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ P[pre + "k"].T).view(T, H, D)
    v = (h @ P[pre + "v"].T).view(T, H, V)
    gi = h @ P[pre + "i"].T + P[pre + "i.b"]
    gf = h @ P[pre + "f"].T + P[pre + "f.b"]
    li = cap * torch.tanh(gi / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh(gf / cap))
    S = torch.zeros(H, D, V)
    n = torch.zeros(H, D)
    m = torch.zeros(H)
    outs = []
    for t in range(T):
        m_new = torch.maximum(lf[t] + m, li[t])
        a = torch.exp(lf[t] + m - m_new)
        b = torch.exp(li[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * (
            k[t][:, :, None] * v[t][:, None, :])
        n = a[:, None] * n + b[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        outs.append(num / den[:, None])
    o = torch.stack(outs)                                   # [T, H, V]
    o = unit_rms(o, eps).reshape(T, H * V) * P[pre + "norm"]
    o = o * torch.sigmoid(h @ P[pre + "g"].T)
    return o @ P[pre + "o"].T


def diff_attention_kv(h, P, pre, mc):
    """Keys [T, G, 2, D] and values [T, G, V] of a layer that owns them."""
    G, D, V = mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    return ((h @ P[pre + "k"].T).view(T, G, 2, D),
            (h @ P[pre + "v"].T).view(T, G, V))


def diff_attention_sequence(h, k, v, P, pre, mc, eps):
    """Differential attention of one sequence over given keys/values."""
    H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q = (h @ P[pre + "q"].T).view(T, H, 2, D)
    lam = (torch.exp((P[pre + "lq1"] * P[pre + "lk1"]).sum())
           - torch.exp((P[pre + "lq2"] * P[pre + "lk2"]).sum())
           + mc["diff"])
    out = torch.zeros(T, H, V)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            maps = []
            for mp in range(2):
                sc = (k[:t + 1, g, mp] @ q[t, hh, mp]) * mc["scale"]
                maps.append(torch.softmax(sc, 0) @ v[:t + 1, g])
            o = maps[0] - lam * maps[1]
            out[t, hh] = unit_rms(o, eps) * (1.0 - mc["diff"])
    return out.reshape(T, H * V) @ P[pre + "o"].T


# ------------------------------------------------------------ feed-forward
def moe_route(h, P, pre, rc):
    """Per token: (chosen experts, their weights)."""
    z = h @ P[pre + "router"].T
    s = torch.softmax(z, -1)
    E, top = rc["experts"], rc["top"]
    cnt, keep = rc["groups"]["count"], rc["groups"]["keep"]
    per = E // cnt
    chosen, weights = [], []
    for t in range(h.shape[0]):
        gs = [max(float(s[t, g * per + j]) for j in range(per))
              for g in range(cnt)]
        kept = sorted(range(cnt), key=lambda g: -gs[g])[:keep]
        allowed = [e for e in range(E) if e // per in kept]
        pick = sorted(allowed, key=lambda e: -float(s[t, e]))[:top]
        w = torch.stack([s[t, e] for e in pick])
        w = w / (w.sum() + 1e-20) * rc["scale"]
        chosen.append(pick)
        weights.append(w)
    return chosen, weights


def moe_ffn(h, P, pre, mlp):
    chosen, weights = moe_route(h, P, pre, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t], weights[t]):
            a = torch.relu(P[f"{pre}e{e}.up"] @ h[t]) ** 2
            out[t] += w * (P[f"{pre}e{e}.down"] @ a)
    return out


# ------------------------------------------------------------- whole model
def forward(tokens, P, cfg, return_layers=False):
    """Logits [T, vocab] of one sequence (and, optionally, the summed
    streams after every layer)."""
    eps = cfg["norm"]["eps"]
    ns = cfg["streams"]
    x0 = P["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = [x0.clone() for _ in range(ns)]
    kv = {}
    per_layer = []

    def sublayer(xs, li, q, fn):
        hc = f"l{li}.hc{q}."
        u = sum(P[hc + "in"][s] * xs[s] for s in range(ns))
        y = fn(dyt(u, P, f"l{li}.norm{q}"))
        return [sum(P[hc + "mix"][s, t] * xs[s] for s in range(ns))
                + P[hc + "out"][t] * y for t in range(ns)]

    for li, lc in enumerate(cfg["layers"]):
        pre, mc = f"l{li}.mix.", lc["mixer"]
        if lc["type"] == "mlstm":
            fn = lambda h: mlstm_sequence(h, P, pre, mc, eps)
        elif lc["type"] == "attention":
            def fn(h, li=li, pre=pre, mc=mc):
                src = mc.get("kv_from")
                if src is None:
                    kv[li] = diff_attention_kv(h, P, pre, mc)
                    src = li
                return diff_attention_sequence(h, *kv[src], P, pre, mc, eps)
        else:
            raise ValueError(lc["type"])
        xs = sublayer(xs, li, 1, fn)
        if lc.get("mlp") is not None:
            xs = sublayer(xs, li, 2,
                          lambda h: moe_ffn(h, P, f"l{li}.mlp.", lc["mlp"]))
        per_layer.append(sum(xs))
    x = dyt(sum(xs), P, "final.norm")
    logits = x @ P["head"].T
    return (logits, torch.stack(per_layer)) if return_layers else logits
