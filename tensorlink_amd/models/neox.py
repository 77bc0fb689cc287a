"""GPT-NeoX / Pythia model family.

Proves the zoo extends beyond the Llama shape (the reference auto-stages ANY HF causal LM via its AST injector,
``tensorlink/ml/injector.py:79-90``): LayerNorm with bias (not RMSNorm),
PARALLEL attention+MLP residual (x + attn(ln1 x) + mlp(ln2 x)), partial
rotary embeddings (``rotary_pct`` of each head rotated, the rest passed
through), an ungated GELU MLP, and biases on every linear. Same stage
interface as :class:`~tensorlink_amd.models.dense.StageModel`, so the
pipeline runtime, batcher and trainer drive it unchanged; attention runs
on the shared CDNA4 kernels (head_dim 64/128).
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from tensorlink_amd import ops
from tensorlink_amd.models.configs import ModelConfig
from tensorlink_amd.models.dense import KVCache, TLLinear, compute_inv_freq


class NeoxAttention(nn.Module):
    def __init__(self, config: ModelConfig):
        super().__init__()
        h = config.hidden_size
        self.query_key_value = TLLinear(h, 3 * config.q_size, bias=True)
        self.dense = TLLinear(config.q_size, h, bias=True)
        self.n_heads = config.num_attention_heads
        self.head_dim = config.head_dim
        self.rot = max(2, int(self.head_dim * config.rotary_pct)) // 2 * 2
        self.scale = 1.0 / math.sqrt(self.head_dim)
        self.register_buffer(
            "inv_freq", compute_inv_freq(config)[: self.rot // 2],
            persistent=False)

    def _rope(self, q, k, positions, inverse=False):
        """Partial rotary: rotate the first ``rot`` dims of each head
        in-place, pass the rest through. q/k [T, H, D]."""
        rot = self.rot
        if rot >= self.head_dim:
            ops.apply_rope_(q, k, positions, self.inv_freq,
                            -1.0 if inverse else 1.0)
            return q, k
        qr = q[..., :rot].contiguous()
        kr = k[..., :rot].contiguous()
        ops.apply_rope_(qr, kr, positions, self.inv_freq,
                        -1.0 if inverse else 1.0)
        q = torch.cat([qr, q[..., rot:]], dim=-1)
        k = torch.cat([kr, k[..., rot:]], dim=-1)
        return q, k

    def forward(self, x, positions, kv_cache: Optional[KVCache],
                layer_idx: int, training: bool):
        B, S, H = x.shape
        qkv = self.query_key_value(x)
        # HF NeoX packs qkv per head as [head][q|k|v]; the loader
        # de-interleaves to [q_all | k_all | v_all] rows (native layout)
        q, k, v = qkv.split(self.n_heads * self.head_dim, dim=-1)
        q = q.reshape(B * S, self.n_heads, self.head_dim).contiguous()
        k = k.reshape(B * S, self.n_heads, self.head_dim).contiguous()
        v = v.reshape(B, S, self.n_heads, self.head_dim)
        flat_pos = positions.reshape(-1)
        if training:
            q, k = ops.apply_rope(q, k, flat_pos, self.inv_freq) \
                if self.rot >= self.head_dim else self._rope_train(
                    q, k, flat_pos)
            q = q.view(B, S, self.n_heads, -1)
            k = k.view(B, S, self.n_heads, -1)
            out = ops.attention_train(q, k, v, causal=True,
                                      scale=self.scale)
            return self.dense(out.reshape(B, S, -1))
        q, k = self._rope(q, k, flat_pos)
        q = q.view(B, S, self.n_heads, self.head_dim)
        k = k.view(B, S, self.n_heads, self.head_dim)
        if kv_cache is None:
            out = ops.attention_prefill(q.contiguous(), k.contiguous(),
                                        v.contiguous(), causal=True,
                                        scale=self.scale)
            return self.dense(out.reshape(B, S, -1))
        kv_cache.append(layer_idx, k, v, positions)
        table = getattr(kv_cache, "table", None)
        if S == 1:
            out = ops.attention_decode(
                q, kv_cache.k[layer_idx], kv_cache.v[layer_idx],
                kv_cache.seq_lens + 1, scale=self.scale, block_table=table)
        else:
            off = int(kv_cache.seq_lens.max())
            kv_len = off + S
            if table is None:
                k_attn = kv_cache.k[layer_idx][:, :, :kv_len].permute(
                    0, 2, 1, 3).contiguous()
                v_attn = kv_cache.v[layer_idx][:, :, :kv_len].permute(
                    0, 2, 1, 3).contiguous()
            else:
                k_attn, v_attn = kv_cache.gather_contiguous(layer_idx,
                                                            kv_len)
            out = ops.attention_prefill(q.contiguous(), k_attn, v_attn,
                                        causal=True, scale=self.scale,
                                        q_off=off)
        return self.dense(out.reshape(B, S, -1))

    def _rope_train(self, q, k, flat_pos):
        rot = self.rot
        qr, kr = ops.apply_rope(q[..., :rot].contiguous(),
                                k[..., :rot].contiguous(), flat_pos,
                                self.inv_freq)
        return (torch.cat([qr, q[..., rot:]], -1),
                torch.cat([kr, k[..., rot:]], -1))


class NeoxBlock(nn.Module):
    def __init__(self, config: ModelConfig):
        super().__init__()
        h = config.hidden_size
        self.input_layernorm = nn.LayerNorm(h, eps=config.rms_norm_eps)
        self.post_attention_layernorm = nn.LayerNorm(
            h, eps=config.rms_norm_eps)
        self.attention = NeoxAttention(config)
        self.dense_h_to_4h = TLLinear(h, config.intermediate_size,
                                      bias=True)
        self.dense_4h_to_h = TLLinear(config.intermediate_size, h,
                                      bias=True)
        self.parallel = config.use_parallel_residual

    def _mlp(self, x):
        return self.dense_4h_to_h(
            F.gelu(self.dense_h_to_4h(x), approximate="tanh"))

    def forward(self, x, positions, kv_cache, layer_idx, training):
        attn = self.attention(self.input_layernorm(x), positions, kv_cache,
                              layer_idx, training)
        if self.parallel:
            # x + attn(ln1 x) + mlp(ln2 x) — NeoX parallel residual
            return x + attn + self._mlp(self.post_attention_layernorm(x))
        x = x + attn
        return x + self._mlp(self.post_attention_layernorm(x))


class NeoxStageModel(nn.Module):
    """GPT-NeoX stage with the StageModel interface."""

    def __init__(self, config: ModelConfig, layer_start: int, layer_end: int,
                 has_embedding: bool, has_head: bool):
        super().__init__()
        self.config = config
        self.layer_start = layer_start
        self.layer_end = layer_end
        self.has_embedding = has_embedding
        self.has_head = has_head
        if has_embedding:
            self.embed_in = nn.Embedding(config.vocab_size,
                                         config.hidden_size)
        self.layers = nn.ModuleList(
            [NeoxBlock(config) for _ in range(layer_end - layer_start)])
        if has_head:
            self.final_layer_norm = nn.LayerNorm(config.hidden_size,
                                                 eps=config.rms_norm_eps)
            if not (config.tie_word_embeddings and has_embedding):
                self.embed_out = TLLinear(config.hidden_size,
                                          config.vocab_size, bias=False)

    @property
    def num_layers(self):
        return len(self.layers)

    def make_kv_cache(self, batch, max_seq, device, dtype=None,
                      kv_mode: str = "contiguous"):
        if dtype is None:
            dtype = next(self.parameters()).dtype
        if kv_mode == "paged":
            from tensorlink_amd.models.paged import PagedKVCache
            return PagedKVCache(self.num_layers, batch, max_seq,
                                self.config, device, dtype)
        return KVCache(self.num_layers, batch, max_seq, self.config,
                       device, dtype)

    def head(self, hidden):
        h = self.final_layer_norm(hidden)
        if self.config.tie_word_embeddings and self.has_embedding:
            return h @ self.embed_in.weight.t()
        return self.embed_out(h)

    def forward(self, hidden_or_ids, positions, kv_cache=None,
                training=False, return_logits=True):
        if self.has_embedding and hidden_or_ids.dtype in (torch.int32,
                                                          torch.int64):
            hidden = self.embed_in(hidden_or_ids)
        else:
            hidden = hidden_or_ids
        for i, layer in enumerate(self.layers):
            hidden = layer(hidden, positions, kv_cache, i, training)
        if kv_cache is not None:
            kv_cache.advance(hidden.shape[1])
        if self.has_head and return_logits:
            return self.head(hidden)
        return hidden


def deinterleave_neox_qkv(w: torch.Tensor, n_heads: int,
                          head_dim: int) -> torch.Tensor:
    """HF NeoX query_key_value rows are [head0 q|k|v, head1 q|k|v, ...];
    the native layout is [all q | all k | all v]. Works for weight
    [3h, h] and bias [3h]."""
    rest = w.shape[1:]
    return (w.reshape(n_heads, 3, head_dim, *rest)
            .transpose(0, 1).reshape(3 * n_heads * head_dim, *rest)
            .contiguous())


def load_neox_hf_weights(stage: NeoxStageModel, ckpt_dir: str,
                         dtype=torch.float32) -> int:
    """Map HF GPT-NeoX checkpoint keys (gpt_neox.layers.N.*, interleaved
    qkv) onto the native stage."""
    import os

    from safetensors import safe_open
    path = os.path.join(ckpt_dir, "model.safetensors")
    params = dict(stage.named_parameters())
    cfg = stage.config
    loaded = 0
    with safe_open(path, framework="pt", device="cpu") as f:
        for key in f.keys():
            k = key[len("gpt_neox."):] if key.startswith("gpt_neox.") \
                else key
            native = None
            if k == "embed_in.weight" and stage.has_embedding:
                native = "embed_in.weight"
            elif k.startswith("final_layer_norm.") and stage.has_head:
                native = k
            elif k == "embed_out.weight" and stage.has_head:
                native = "embed_out.weight"
            elif k.startswith("layers."):
                _, idx, rest = k.split(".", 2)
                idx = int(idx)
                if stage.layer_start <= idx < stage.layer_end:
                    rest = rest.replace("mlp.dense_h_to_4h",
                                        "dense_h_to_4h")
                    rest = rest.replace("mlp.dense_4h_to_h",
                                        "dense_4h_to_h")
                    native = f"layers.{idx - stage.layer_start}.{rest}"
            if native and native in params:
                t = f.get_tensor(key).to(dtype)
                if "query_key_value" in native:
                    t = deinterleave_neox_qkv(
                        t, cfg.num_attention_heads, cfg.head_dim)
                with torch.no_grad():
                    params[native].copy_(t)
                loaded += 1
    return loaded
