"""Plain token-by-token oracle of the Senulix design, written from its
equations only: one function per mechanism, float64 throughout, no cache,
no batching, nothing shared with the serving path.

A model is (cfg, W): ``cfg`` the dictionary of config.json and ``W`` a
dictionary tensor name -> torch tensor (any float dtype; tables as given).
"""

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate(x, pos, dims, base):
    """x [..., d] at one position: the first ``dims`` entries are rotated
    in pairs (i, i + dims/2); the others pass."""
    half = dims // 2
    out = x.clone()
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * math.cos(a) - v * math.sin(a)
        out[..., i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def lightning(h, P, mc, eps):
    """h [T, W] -> [T, W]: decayed outer-product memory per head."""
    H, D, V = mc["heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q = silu(h @ P["q"].T).view(T, H, D)
    k = silu(h @ P["k"].T).view(T, H, D)
    v = silu(h @ P["v"].T).view(T, H, V)
    S = torch.zeros(H, D, V, dtype=F64)
    o = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        for hd in range(H):
            S[hd] = mc["decay"][hd] * S[hd] + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    y = rms(o.reshape(T, H * V), eps) * P["norm"]
    y = y * torch.sigmoid(h @ P["g"].T)
    return y @ P["o"].T


def latent_kv(h, P, mc, eps):
    """What a latent layer caches: (c [T, rank], rotated shared key
    [T, rot_dim])."""
    R, rd = mc["kv_rank"], mc["rot_dim"]
    d = h @ P["dkv"].T
    c = rms(d[:, :R], eps) * P["dkv.norm"]
    kr = torch.stack([rotate(d[t, R:], t, mc["rot"]["dims"],
                             mc["rot"]["base"]) for t in range(d.shape[0])])
    assert rd == mc["rot"]["dims"]
    return c, kr


def latent_attention(h, P, mc, eps, shared=None):
    H, D, rd, V = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"]
    T = h.shape[0]
    c, kr = shared if shared is not None else latent_kv(h, P, mc, eps)
    q = (h @ P["q"].T).view(T, H, D + rd)
    ku = (c @ P["uk"].T).view(T, H, D)
    vv = (c @ P["uv"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        for hd in range(H):
            qr = rotate(q[t, hd, D:], t, mc["rot"]["dims"],
                        mc["rot"]["base"])
            s = torch.stack([(q[t, hd, :D] @ ku[j, hd] + qr @ kr[j])
                             * mc["scale"] for j in range(t + 1)])
            p = torch.softmax(s, 0)
            o[t, hd] = p @ vv[:t + 1, hd]
    return o.reshape(T, H * V) @ P["o"].T, (c, kr)


def window_attention(h, P, mc, eps):
    H, G, D, V = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    win = mc["mask"]["size"]
    q = rms(h @ P["q"].T, eps) * P["q.norm"]
    k = rms(h @ P["k"].T, eps) * P["k.norm"]
    v = (h @ P["v"].T).view(T, G, V)
    q = q.view(T, H, D)
    k = k.view(T, G, D)
    rot = mc["rot"]
    q = torch.stack([rotate(q[t], t, rot["dims"], rot["base"])
                     for t in range(T)])
    k = torch.stack([rotate(k[t], t, rot["dims"], rot["base"])
                     for t in range(T)])
    o = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        lo = max(0, t - win + 1)
        s = torch.zeros(H, t + 1 - lo, dtype=F64)
        for hd in range(H):
            g = hd // (H // G)
            s[hd] = (k[lo:t + 1, g] @ q[t, hd]) * mc["scale"]
        s = P["talk"] @ s                        # mix the heads' scores
        e = torch.exp(s)
        p = e / (1.0 + e.sum(-1, keepdim=True))  # a sink of score 0
        for hd in range(H):
            o[t, hd] = p[hd] @ v[lo:t + 1, hd // (H // G)]
    return o.reshape(T, H * V) @ P["o"].T


def dense_ff(h, P):
    return gelu_erf(h @ P["up"].T) @ P["down"].T


def token_side(x, tokens, i, W, cfg):
    dim = cfg["token_side"]["dim"]
    eps = cfg["norm"]["eps"]
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return x + rms(y, eps) * W[f"l{i}.side.norm"]


def forward(cfg, W, tokens, layer_out=None):
    """Logits [T, vocab] for one sequence from position 0; ``layer_out``
    (a list) receives the residual after every layer."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = W["embed"][tokens]
    shared = {}
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        P = {k[len(f"l{i}.mix."):]: v for k, v in W.items()
             if k.startswith(f"l{i}.mix.")}
        if lc["type"] == "lightning":
            y = lightning(x, P, mc, eps)
        elif lc["type"] == "latent_attention":
            src = mc.get("kv_from")
            y, kv = latent_attention(x, P, mc, eps,
                                     None if src is None else shared[src])
            shared[i] = kv
        elif lc["type"] == "attention":
            y = window_attention(x, P, mc, eps)
        else:
            raise KeyError(lc["type"])
        x = x + rms(y, eps) * (1.0 + W[f"l{i}.norm1"])
        if lc.get("mlp") is not None:
            assert lc["mlp"]["kind"] == "dense"
            y = dense_ff(x, {"up": W[f"l{i}.mlp.up"],
                             "down": W[f"l{i}.mlp.down"]})
            x = x + rms(y, eps) * (1.0 + W[f"l{i}.norm2"])
        if cfg.get("token_side"):
            x = token_side(x, tokens, i, W, cfg)
        if layer_out is not None:
            layer_out.append(x.clone())
    z = (rms(x, eps) * (1.0 + W["final.norm"])) @ W["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * torch.tanh(z / cap)
    return z
