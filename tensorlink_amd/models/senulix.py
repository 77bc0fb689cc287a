"""Senulix model family: a layered decoder whose ``config.json`` lists
every layer — lightning (decayed linear) attention, latent attention
(optionally reading an earlier layer's cached latents) or windowed
attention with score mixing and a sink — followed by an optional dense
GELU feed-forward and a per-layer token input. The norm sits on every
sublayer's OUTPUT: x <- x + norm(sublayer(x)); the residual is fp32.

The blocks live in :mod:`tensorlink_amd.models.mixers`; this file reads
the configuration, assembles them, maps checkpoint tensor names and runs
the stage over a flat ragged batch through the stage interface of
:class:`~tensorlink_amd.models.layered.LayeredStage`. The residual stays
fp32 between layers, so the family runs as ONE stage (PP = 1).
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
from tensorlink_amd.models.mixers import (DenseFF, LatentAttention,
                                          LightningMixer, RMSWeight,
                                          TokenSide, WindowAttention)
from tensorlink_amd.ops import mixers as mx

MIXERS = ("lightning", "latent_attention", "attention")


@dataclass
class SenulixConfig(ModelConfig):
    """Flat ModelConfig fields are filled for the planner and the engine;
    ``layer_specs`` (the checkpoint's ``layers`` list) is authoritative."""
    layer_specs: List[dict] = field(default_factory=list)
    side_dim: int = 0                   # per-layer token input; 0 = none
    logit_softcap: float = 0.0          # 0 = none
    architecture: str = "senulix"

    @classmethod
    def from_dict(cls, cfg: dict, name: str = "senulix") -> "SenulixConfig":
        if "layer_specs" in cfg:                     # own to_json round trip
            known = {f.name for f in cls.__dataclass_fields__.values()}
            return cls(**{k: v for k, v in cfg.items() if k in known})
        layers = cfg["layers"]
        for i, lc in enumerate(layers):
            if lc["type"] not in MIXERS:
                raise KeyError(f"layer {i}: unknown mixer {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise KeyError(f"layer {i}: unknown feed-forward "
                               f"{mlp.get('kind')!r}")
            mc = lc["mixer"]
            src = mc.get("kv_from")
            if src is not None:
                if lc["type"] != "latent_attention":
                    raise KeyError(f"layer {i}: kv_from is a latent-"
                                   "attention option")
                sm = layers[src]["mixer"] if 0 <= src < i else None
                if (sm is None or layers[src]["type"] != "latent_attention"
                        or sm.get("kv_from") is not None
                        or sm["kv_rank"] != mc["kv_rank"]
                        or sm["rot_dim"] != mc["rot_dim"]
                        or sm["rot"] != mc["rot"]):
                    raise KeyError(f"layer {i}: kv_from must name an "
                                   "earlier latent layer with its own "
                                   "latents and the same rank and rotation")
            if lc["type"] == "latent_attention" and \
                    mc["rot"]["dims"] != mc["rot_dim"]:
                raise KeyError(f"layer {i}: the rotated part is rot_dim wide")
            if lc["type"] == "lightning" and len(mc["decay"]) != mc["heads"]:
                raise KeyError(f"layer {i}: one decay per head")
        heads = max(lc["mixer"]["heads"] for lc in layers)
        kvh = max(lc["mixer"].get("kv_heads", 1) for lc in layers)
        dim = max(lc["mixer"]["dim"] for lc in layers)
        inter = max((lc["mlp"]["ff"] for lc in layers
                     if lc.get("mlp") is not None), default=cfg["width"])
        side = cfg.get("token_side") or {}
        return cls(
            name=name, vocab_size=cfg["vocab"], hidden_size=cfg["width"],
            intermediate_size=inter, num_hidden_layers=len(layers),
            num_attention_heads=heads, num_key_value_heads=kvh,
            head_dim=dim, rms_norm_eps=cfg["norm"]["eps"],
            tie_word_embeddings=False, layer_specs=layers,
            side_dim=int(side.get("dim", 0)),
            logit_softcap=float(cfg.get("logit_softcap") or 0.0))

    def param_count(self, include_embeddings: bool = True) -> int:
        w = self.hidden_size
        total = w
        for lc in self.layer_specs:
            mc = lc["mixer"]
            H, D, V = mc["heads"], mc["dim"], mc["vdim"]
            total += w + H * V * w
            if lc["type"] == "lightning":
                total += w * (2 * H * D + 2 * H * V) + H * V
            elif lc["type"] == "latent_attention":
                R, rd = mc["kv_rank"], mc["rot_dim"]
                total += w * H * (D + rd) + H * (D + V) * R
                if mc.get("kv_from") is None:
                    total += w * (R + rd) + R
            else:
                G = mc["kv_heads"]
                total += w * (H * D + G * D + G * V) + H * D + G * D + H * H
            if lc.get("mlp") is not None:
                total += w + 2 * w * lc["mlp"]["ff"]
            if self.side_dim:
                total += 2 * w * self.side_dim + w
        if include_embeddings:
            total += self.vocab_size * (2 * w + self.side_dim
                                        * len(self.layer_specs))
        return total


def build_mixer(lc: dict, width: int, eps: float) -> nn.Module:
    mc = lc["mixer"]
    if lc["type"] == "lightning":
        return LightningMixer(width, mc["heads"], mc["dim"], mc["vdim"],
                              mc["decay"], eps)
    if lc["type"] == "latent_attention":
        return LatentAttention(width, mc["heads"], mc["dim"], mc["rot_dim"],
                               mc["vdim"], mc["kv_rank"], mc["scale"],
                               mc["rot"]["base"], eps, mc.get("kv_from"))
    rot = mc.get("rot") or {"dims": 0, "base": 1.0}
    return WindowAttention(width, mc["heads"], mc["kv_heads"], mc["dim"],
                           mc["vdim"], mc["scale"], rot["dims"], rot["base"],
                           (mc.get("mask") or {}).get("size", 0), eps)


class SenulixLayer(nn.Module):
    def __init__(self, config: SenulixConfig, idx: int):
        super().__init__()
        lc = config.layer_specs[idx]
        w, eps = config.hidden_size, config.rms_norm_eps
        self.mix = build_mixer(lc, w, eps)
        self.norm1 = RMSWeight(w, one_plus=True)
        self.mlp = None
        if lc.get("mlp") is not None:
            self.mlp = DenseFF(w, lc["mlp"]["ff"])
            self.norm2 = RMSWeight(w, one_plus=True)
        self.side = None
        if config.side_dim:
            self.side = TokenSide(w, config.side_dim, idx * config.side_dim)


class SenulixStageModel(LayeredStage):
    """Whole-model stage (embeddings, every layer, final norm + head)."""

    def __init__(self, config: SenulixConfig, layer_start: int,
                 layer_end: int, has_embedding: bool, has_head: bool):
        super().__init__()
        if not (has_embedding and has_head and layer_start == 0
                and layer_end == config.num_hidden_layers):
            raise ValueError("the Senulix family runs as a single stage "
                             "(fp32 residual); use world=1")
        self.config = config
        self.layer_start, self.layer_end = layer_start, layer_end
        self.has_embedding = self.has_head = True
        n = config.num_hidden_layers
        self.embed_tokens = nn.Embedding(config.vocab_size,
                                         config.hidden_size)
        self.side_embed = (nn.Embedding(config.vocab_size,
                                        n * config.side_dim)
                           if config.side_dim else None)
        self.layers = nn.ModuleList([SenulixLayer(config, i)
                                     for i in range(n)])
        self.norm = RMSWeight(config.hidden_size, one_plus=True)
        self.lm_head = TLLinear(config.hidden_size, config.vocab_size,
                                bias=False)
        self.layer_sums = None      # list -> residual after every layer

    def head(self, hidden: torch.Tensor) -> torch.Tensor:
        """Final norm, vocabulary projection and soft cap of residual rows
        [..., W] (fp32); fp32 logits."""
        shape = hidden.shape
        x = hidden.reshape(-1, shape[-1]).float()
        h = mx.rms_scale(x, self.norm.w32(), self.config.rms_norm_eps, True,
                         out_dtype=self.lm_head.weight.dtype)
        z = self.lm_head(h).float()
        if self.config.logit_softcap:
            z = mx.soft_cap_(z, self.config.logit_softcap)
        return z.reshape(*shape[:-1], -1)

    @torch.no_grad()
    def forward(self, hidden_or_ids, positions, kv_cache=None,
                training: bool = False, return_logits: bool = True):
        if training:
            raise NotImplementedError(
                "the Senulix family is served, not trained, by this build")
        B, S = hidden_or_ids.shape[:2]
        dev = hidden_or_ids.device
        dtype = self.lm_head.weight.dtype
        eps = self.config.rms_norm_eps
        if kv_cache is None:
            kv_cache = self.make_kv_cache(B, int(positions.max()) + 1, dev,
                                          dtype)
        meta = self._meta(kv_cache, positions, B, S)
        tokens = hidden_or_ids.reshape(-1)
        X = self.embed_tokens(tokens).float().contiguous()
        h = X if dtype == torch.float32 else X.to(dtype)
        table = self.side_embed.weight if self.side_embed is not None \
            else None
        tok32 = tokens.to(torch.int32) if table is not None else None
        for li, layer in enumerate(self.layers):
            y = layer.mix(h, meta, kv_cache, li)
            h = mx.postnorm_add(X, y, layer.norm1.w32(), eps, True, dtype)
            if layer.mlp is not None:
                h = mx.postnorm_add(X, layer.mlp(h), layer.norm2.w32(), eps,
                                    True, dtype)
            if layer.side is not None:
                h = mx.postnorm_add(X, layer.side(h, table, tok32),
                                    layer.side.norm.w32(), eps, False, dtype)
            if self.layer_sums is not None:
                self.layer_sums.append(X.clone())
        if kv_cache is not None:
            kv_cache.advance(S)
        u = X.view(B, S, -1)
        return self.head(u) if return_logits else u


# ------------------------------------------------------------------ weights
def _name_map(stage: SenulixStageModel):
    """checkpoint tensor name -> (parameter, row offset)."""
    P = dict(stage.named_parameters())
    m = {"embed": ("embed_tokens.weight", 0), "head": ("lm_head.weight", 0),
         "final.norm": ("norm.weight", 0)}
    if stage.side_embed is not None:
        m["side.embed"] = ("side_embed.weight", 0)
    for i, layer in enumerate(stage.layers):
        a, b = f"l{i}.", f"layers.{i}."
        m[f"{a}norm1"] = (f"{b}norm1.weight", 0)
        mix = layer.mix
        if mix.kind == "lightning":
            for nm, off in zip("qkvg", mix.offs):
                m[f"{a}mix.{nm}"] = (f"{b}mix.proj.weight", off)
            m[f"{a}mix.norm"] = (f"{b}mix.norm", 0)
        elif mix.kind == "latent_attention":
            m[f"{a}mix.q"] = (f"{b}mix.qdkv.weight", 0)
            if mix.kv_from is None:
                m[f"{a}mix.dkv"] = (f"{b}mix.qdkv.weight", mix.q_cols)
                m[f"{a}mix.dkv.norm"] = (f"{b}mix.dkv_norm", 0)
            m[f"{a}mix.uk"] = (f"{b}mix.uk", 0)
            m[f"{a}mix.uv"] = (f"{b}mix.uv", 0)
        else:
            m[f"{a}mix.q"] = (f"{b}mix.qkv.weight", 0)
            m[f"{a}mix.k"] = (f"{b}mix.qkv.weight", mix.q_cols)
            m[f"{a}mix.v"] = (f"{b}mix.qkv.weight", mix.q_cols + mix.k_cols)
            m[f"{a}mix.q.norm"] = (f"{b}mix.q_norm", 0)
            m[f"{a}mix.k.norm"] = (f"{b}mix.k_norm", 0)
            m[f"{a}mix.talk"] = (f"{b}mix.talk", 0)
        m[f"{a}mix.o"] = (f"{b}mix.o_proj.weight", 0)
        if layer.mlp is not None:
            m[f"{a}norm2"] = (f"{b}norm2.weight", 0)
            m[f"{a}mlp.up"] = (f"{b}mlp.up.weight", 0)
            m[f"{a}mlp.down"] = (f"{b}mlp.down.weight", 0)
        if layer.side is not None:
            m[f"{a}side.gate"] = (f"{b}side.gate.weight", 0)
            m[f"{a}side.proj"] = (f"{b}side.proj.weight", 0)
            m[f"{a}side.norm"] = (f"{b}side.norm.weight", 0)
    return m, P


@torch.no_grad()
def load_senulix_weights(stage: SenulixStageModel, ckpt_dir: str,
                         dtype=torch.bfloat16) -> int:
    """Fill the stage from ``model.safetensors``; every tensor of the
    checkpoint must be consumed and every parameter filled."""
    names, P = _name_map(stage)
    return load_named_tensors(P, names, ckpt_dir)


@torch.no_grad()
def init_senulix_random(stage: SenulixStageModel, seed: int = 0) -> None:
    """Scaled-normal matrices, norm weights near their neutral value,
    near-identity score mixing: finite activations at any depth for
    benchmarks and tests."""
    g = torch.Generator().manual_seed(seed)
    for name, p in stage.named_parameters():
        t = torch.empty(p.shape, dtype=torch.float32)
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith((".norm1.weight", ".norm2.weight")) \
                or name == "norm.weight":
            t = 0.1 * torch.randn(p.shape, generator=g)
        elif leaf in ("q_norm", "k_norm", "dkv_norm", "norm") \
                or name.endswith("side.norm.weight"):
            t = 1.0 + 0.1 * torch.randn(p.shape, generator=g)
        elif leaf == "talk":
            n = p.shape[0]
            t = torch.eye(n) + 0.2 * torch.randn(n, n, generator=g)
        elif name in ("embed_tokens.weight", "side_embed.weight"):
            t.normal_(0.0, 1.0, generator=g)
        else:
            t.normal_(0.0, 1.0 / math.sqrt(p.shape[-1]), generator=g)
        p.copy_(t.to(p.dtype))


def read_config(path: str) -> Optional[SenulixConfig]:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    if cfg.get("architecture") in ("Senulix", "senulix"):
        return SenulixConfig.from_dict(cfg, name=path)
    return None
