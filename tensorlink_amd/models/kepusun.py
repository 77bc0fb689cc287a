"""Kepusun model family: a layered decoder whose ``config.json`` lists
every layer — a matrix-memory (mLSTM) or differential-attention mixer,
optionally followed by a group-limited mixture of experts — under
Dynamic-Tanh norms and hyper-connected residual streams.

The blocks live in :mod:`tensorlink_amd.models.mixers`; this file only
reads the configuration, assembles them, maps checkpoint tensor names and
runs the stage over a flat ragged batch. It keeps the stage interface of
:class:`~tensorlink_amd.models.dense.StageModel` (embed / forward / head /
make_kv_cache), so the runner, the continuous batcher and the engine drive
it like the other families. The residual is ``streams`` fp32 copies, which
do not fit the [B, S, H] inter-stage activation of the pipeline runtime:
the family runs as ONE stage (PP = 1).
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import List, Optional

import torch
import torch.nn as nn

from tensorlink_amd.models.configs import ModelConfig
from tensorlink_amd.models.dense import TLLinear
from tensorlink_amd.models.layered import LayeredStage, load_named_tensors
from tensorlink_amd.models.mixers import (DiffAttention, DynamicTanh,
                                          GroupLimitedMoE, HyperConnection,
                                          MLSTMMixer)
from tensorlink_amd.ops import mixers as mx


@dataclass
class KepusunConfig(ModelConfig):
    """Flat ModelConfig fields are filled for the planner and the engine;
    ``layer_specs`` (the checkpoint's ``layers`` list) is authoritative."""
    layer_specs: List[dict] = field(default_factory=list)
    streams: int = 1
    architecture: str = "kepusun"

    @classmethod
    def from_dict(cls, cfg: dict, name: str = "kepusun") -> "KepusunConfig":
        if "layer_specs" in cfg:                     # own to_json round trip
            known = {f.name for f in cls.__dataclass_fields__.values()}
            return cls(**{k: v for k, v in cfg.items() if k in known})
        layers = cfg["layers"]
        for i, lc in enumerate(layers):
            if lc["type"] not in ("mlstm", "attention"):
                raise KeyError(f"layer {i}: unknown mixer {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") != "moe":
                raise KeyError(f"layer {i}: unknown feed-forward "
                               f"{mlp.get('kind')!r}")
            src = lc["mixer"].get("kv_from")
            if src is not None:
                sm = layers[src]["mixer"] if 0 <= src < i else None
                if (sm is None or layers[src]["type"] != "attention"
                        or sm.get("kv_from") is not None):
                    raise KeyError(f"layer {i}: kv_from must name an "
                                   "earlier attention layer with its own "
                                   "keys and values")
        heads = max(lc["mixer"]["heads"] for lc in layers)
        kvh = max(lc["mixer"].get("kv_heads", lc["mixer"]["heads"])
                  for lc in layers)
        dim = max(lc["mixer"]["dim"] for lc in layers)
        moes = [lc["mlp"] for lc in layers if lc.get("mlp") is not None]
        inter = max((m["expert"]["ff"] * m["router"]["experts"]
                     for m in moes), default=cfg["width"])
        return cls(
            name=name, vocab_size=cfg["vocab"], hidden_size=cfg["width"],
            intermediate_size=inter, num_hidden_layers=len(layers),
            num_attention_heads=heads, num_key_value_heads=kvh,
            head_dim=dim, rms_norm_eps=cfg["norm"]["eps"],
            tie_word_embeddings=False, layer_specs=layers,
            streams=int(cfg.get("streams", 1)))

    def param_count(self, include_embeddings: bool = True) -> int:
        w, ns = self.hidden_size, self.streams
        total = 2 * w + 1
        for lc in self.layer_specs:
            mc = lc["mixer"]
            H, D, V = mc["heads"], mc["dim"], mc["vdim"]
            total += 2 * w + 1 + 2 * ns + ns * ns
            if lc["type"] == "mlstm":
                total += w * (2 * H * D + 2 * H * V) + H * V * w + H * V
                total += 2 * H * (w + 1)
            else:
                total += w * H * 2 * D + H * V * w + 4 * D
                if mc.get("kv_from") is None:
                    total += w * mc["kv_heads"] * (2 * D + V)
            mlp = lc.get("mlp")
            if mlp is not None:
                E = mlp["router"]["experts"]
                total += 2 * w + 1 + 2 * ns + ns * ns
                total += E * w + 2 * E * w * mlp["expert"]["ff"]
        if include_embeddings:
            total += 2 * self.vocab_size * w
        return total


class KepusunLayer(nn.Module):
    def __init__(self, config: KepusunConfig, idx: int):
        super().__init__()
        lc = config.layer_specs[idx]
        mc = lc["mixer"]
        w, eps, ns = config.hidden_size, config.rms_norm_eps, config.streams
        self.norm1 = DynamicTanh(w)
        self.hc1 = HyperConnection(ns)
        if lc["type"] == "mlstm":
            self.mix = MLSTMMixer(w, mc["heads"], mc["dim"], mc["vdim"],
                                  mc["gate_cap"], eps)
        else:
            self.mix = DiffAttention(w, mc["heads"], mc["kv_heads"],
                                     mc["dim"], mc["vdim"], mc["scale"],
                                     mc["diff"], eps, mc.get("kv_from"))
        mlp = lc.get("mlp")
        self.mlp = None
        if mlp is not None:
            r = mlp["router"]
            groups = r.get("groups") or {"count": 1, "keep": 1}
            self.norm2 = DynamicTanh(w)
            self.hc2 = HyperConnection(ns)
            self.mlp = GroupLimitedMoE(w, mlp["expert"]["ff"], r["experts"],
                                       r["top"], groups["count"],
                                       groups["keep"], r.get("scale", 1.0))


class KepusunStageModel(LayeredStage):
    """Whole-model stage (embedding, every layer, final norm + head)."""

    def __init__(self, config: KepusunConfig, layer_start: int,
                 layer_end: int, has_embedding: bool, has_head: bool):
        super().__init__()
        if not (has_embedding and has_head and layer_start == 0
                and layer_end == config.num_hidden_layers):
            raise ValueError("the Kepusun family runs as a single stage "
                             "(fp32 multi-stream residual); use world=1")
        self.config = config
        self.layer_start, self.layer_end = layer_start, layer_end
        self.has_embedding = self.has_head = True
        self.embed_tokens = nn.Embedding(config.vocab_size,
                                         config.hidden_size)
        self.layers = nn.ModuleList(
            [KepusunLayer(config, i)
             for i in range(config.num_hidden_layers)])
        self.norm = DynamicTanh(config.hidden_size)
        self.lm_head = TLLinear(config.hidden_size, config.vocab_size,
                                bias=False)
        self.layer_sums = None      # list -> per-layer stream sums (debug)

    # -------------------------------------------------------- forward
    def head(self, hidden: torch.Tensor) -> torch.Tensor:
        """Final Dynamic-Tanh norm + vocabulary projection of summed
        streams [..., W] (fp32)."""
        shape = hidden.shape
        X = hidden.reshape(1, -1, shape[-1]).float().contiguous()
        h, _ = mx.hyper_dyt(X, None, None, None, None, *self.norm.params(),
                            out_dtype=self.lm_head.weight.dtype)
        return self.lm_head(h).reshape(*shape[:-1], -1)

    @torch.no_grad()
    def forward(self, hidden_or_ids, positions, kv_cache=None,
                training: bool = False, return_logits: bool = True):
        if training:
            raise NotImplementedError(
                "the Kepusun family is served, not trained, by this build")
        B, S = hidden_or_ids.shape[:2]
        dev = hidden_or_ids.device
        dtype = self.lm_head.weight.dtype
        if kv_cache is None:
            kv_cache = self.make_kv_cache(B, int(positions.max()) + 1, dev,
                                          dtype)
        meta = self._meta(kv_cache, positions, B, S)
        ns, W = self.config.streams, self.config.hidden_size
        x0 = self.embed_tokens(hidden_or_ids.reshape(-1)).float()
        X = x0.unsqueeze(0).repeat(ns, 1, 1).contiguous()
        pend = (None, None, None)          # (y, mix, out) not yet applied
        for li, layer in enumerate(self.layers):
            subs = [(layer.hc1, layer.norm1, None)]
            if layer.mlp is not None:
                subs.append((layer.hc2, layer.norm2, layer.mlp))
            for hc, norm, mlp in subs:
                h, _ = mx.hyper_dyt(X, *pend, hc._f32("inw"), *norm.params(),
                                    out_dtype=dtype)
                y = (layer.mix(h, meta, kv_cache, li) if mlp is None
                     else mlp(h))
                pend = (y.contiguous(), hc._f32("mix"), hc._f32("out"))
            if self.layer_sums is not None:
                _, u = mx.hyper_dyt(X, *pend, want_sum=True)
                self.layer_sums.append(u)
                pend = (None, None, None)
        _, u = mx.hyper_dyt(X, *pend, want_sum=True)
        if kv_cache is not None:
            kv_cache.advance(S)
        u = u.view(B, S, W)
        return self.head(u) if return_logits else u


# ------------------------------------------------------------------ weights
def _name_map(stage: KepusunStageModel):
    """checkpoint tensor name -> (parameter, row offset, expert index)."""
    P = dict(stage.named_parameters())
    m = {"embed": ("embed_tokens.weight", 0), "head": ("lm_head.weight", 0),
         "final.norm": ("norm.weight", 0), "final.norm.b": ("norm.bias", 0),
         "final.norm.alpha": ("norm.alpha", 0)}
    for i, layer in enumerate(stage.layers):
        a, b = f"l{i}.", f"layers.{i}."
        for q in (1, 2):
            if q == 2 and layer.mlp is None:
                continue
            m[f"{a}norm{q}"] = (f"{b}norm{q}.weight", 0)
            m[f"{a}norm{q}.b"] = (f"{b}norm{q}.bias", 0)
            m[f"{a}norm{q}.alpha"] = (f"{b}norm{q}.alpha", 0)
            m[f"{a}hc{q}.in"] = (f"{b}hc{q}.inw", 0)
            m[f"{a}hc{q}.out"] = (f"{b}hc{q}.out", 0)
            m[f"{a}hc{q}.mix"] = (f"{b}hc{q}.mix", 0)
        mix = layer.mix
        if mix.kind == "mlstm":
            for nm, off in zip("qkvg", mix.offs):
                m[f"{a}mix.{nm}"] = (f"{b}mix.proj.weight", off)
            m[f"{a}mix.i"] = (f"{b}mix.gate.weight", 0)
            m[f"{a}mix.f"] = (f"{b}mix.gate.weight", mix.H)
            m[f"{a}mix.i.b"] = (f"{b}mix.gate.bias", 0)
            m[f"{a}mix.f.b"] = (f"{b}mix.gate.bias", mix.H)
            m[f"{a}mix.norm"] = (f"{b}mix.norm", 0)
        else:
            m[f"{a}mix.q"] = (f"{b}mix.qkv.weight", 0)
            if mix.kv_from is None:
                m[f"{a}mix.k"] = (f"{b}mix.qkv.weight", mix.q_cols)
                m[f"{a}mix.v"] = (f"{b}mix.qkv.weight",
                                  mix.q_cols + mix.k_cols)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                m[f"{a}mix.{nm}"] = (f"{b}mix.{nm}", 0)
        m[f"{a}mix.o"] = (f"{b}mix.o_proj.weight", 0)
        if layer.mlp is not None:
            m[f"{a}mlp.router"] = (f"{b}mlp.router", 0)
            for e in range(layer.mlp.E):
                m[f"{a}mlp.e{e}.up"] = (f"{b}mlp.up", e)
                m[f"{a}mlp.e{e}.down"] = (f"{b}mlp.down", e)
    return m, P


@torch.no_grad()
def load_kepusun_weights(stage: KepusunStageModel, ckpt_dir: str,
                         dtype=torch.bfloat16) -> int:
    """Fill the stage from ``model.safetensors``; every tensor of the
    checkpoint must be consumed and every parameter filled."""
    names, P = _name_map(stage)
    optional = []
    if stage.config.streams == 1:
        # a single stream without hyper-connection tensors is the plain
        # pre-norm residual: the identity defaults stand
        optional = [k for k in P if ".hc" in k
                    and k.rsplit(".", 1)[-1] in ("inw", "out", "mix")]
    return load_named_tensors(P, names, ckpt_dir, optional)


@torch.no_grad()
def init_kepusun_random(stage: KepusunStageModel, seed: int = 0) -> None:
    """Scaled-normal matrices, near-identity stream mixing, small gate and
    lambda vectors: finite activations at any depth for benchmarks/tests."""
    g = torch.Generator().manual_seed(seed)
    w = stage.config.hidden_size
    ns = stage.config.streams
    for name, p in stage.named_parameters():
        t = torch.empty(p.shape, dtype=torch.float32)
        if name.endswith(("hc1.mix", "hc2.mix")):
            t = torch.eye(ns) + 0.05 * torch.randn(ns, ns, generator=g)
        elif name.endswith((".inw",)):
            t = torch.full((ns,), 1.0 / ns) + 0.05 * torch.randn(
                ns, generator=g)
        elif name.endswith((".out",)):
            t = 1.0 + 0.05 * torch.randn(ns, generator=g)
        elif name.endswith(".alpha"):
            t.fill_(0.5)
        elif name.endswith(("norm.weight", "norm1.weight", "norm2.weight",
                            "mix.norm")):
            t = 1.0 + 0.05 * torch.randn(p.shape, generator=g)
        elif name.endswith(".bias"):
            t = 0.05 * torch.randn(p.shape, generator=g)
        elif name.endswith(("lq1", "lk1", "lq2", "lk2")):
            t = 0.3 * torch.randn(p.shape, generator=g)
        elif name == "embed_tokens.weight":
            t.normal_(0.0, 1.0, generator=g)
        else:
            fan_in = p.shape[-1]
            t.normal_(0.0, 1.0 / math.sqrt(fan_in), generator=g)
        p.copy_(t.to(p.dtype))


def read_config(path: str) -> Optional[KepusunConfig]:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    if cfg.get("architecture") in ("Kepusun", "kepusun"):
        return KepusunConfig.from_dict(cfg, name=path)
    return None
