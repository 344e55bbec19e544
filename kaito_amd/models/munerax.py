"""Munerax: a pre-norm latent-attention decoder stack served by the paged
engine.

Every layer is  x ← x + mixer(rms(x)·w₁);  x ← x + ff(rms(x)·w₂)  (the
second half only where the layer has a feed-forward). The stream x is
f32; sub-layers see its norm rounded to the activation dtype. The mixer
is LatentAttention (models/mixers.py): the paged cache holds one
low-rank latent and one rotated key part per token; a layer may read an
earlier layer's cache instead of projecting its own. The feed-forward is
GeluGLU or the engine's MoEMLP with squared-relu experts, group-limited
sigmoid routing and an always-on shared expert.

Input: the scaled token embedding plus a hashed bigram embedding; the
previous token of a sequence is per-sequence state (one int64 per state
slot), so a portion that continues a sequence finds it there. Output:
final norm, then the embedding table as the head.

Each sub-layer's residual add is fused with the NEXT sub-layer's norm
(ops.residual_add_norm), so a layer receives its normed input and is told
the weight of the norm that follows it.
"""
from __future__ import annotations

import math
from typing import Dict

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import ModelConfig
from .hybrid_base import HybridStackBase, MixerLayerBase, f32_vector
from .hybrid_config import LayerSpec, layer_moe_config
from .mixers import GeluGLU, LatentAttention
from .moe import MoEMLP


class MuneraxLayer(MixerLayerBase):
    def __init__(self, cfg: ModelConfig, spec: LayerSpec):
        super().__init__()
        self.cfg, self.spec = cfg, spec
        h, eps, dt = cfg.hidden_size, cfg.rms_eps, cfg.dtype
        if spec.kind != "latent_attention":
            raise ValueError(spec.kind)
        self.attn = LatentAttention(h, spec.latent, dt, eps)
        self.norm1 = f32_vector(h)
        if spec.glu is not None:
            self.mlp = GeluGLU(h, spec.glu, dt)
        elif spec.moe is not None:
            self.mlp = MoEMLP(layer_moe_config(cfg, spec.moe))
        else:
            self.mlp = None
        if self.mlp is not None:
            self.norm2 = f32_vector(h)

    def mixers(self):
        return [self.attn]

    def forward(self, x32, h, positions, cache, meta, next_norm):
        """h = rms(x32)·norm1 in the activation dtype; `cache` is this
        layer's cache or that of the layer whose latents it reads.
        Returns the next layer's normed input (None after the last)."""
        eps, dt = self.cfg.rms_eps, self.cfg.dtype
        after_mixer = self.norm2 if self.mlp is not None else next_norm
        y = self.attn(h, positions, self._view(cache, self.attn), meta)
        h = ops.residual_add_norm(x32, y, after_mixer, eps, dt)
        if self.mlp is not None:
            h = ops.residual_add_norm(x32, self.mlp(h), next_norm, eps, dt)
        return h


class MuneraxForCausalLM(HybridStackBase):
    def __init__(self, cfg: ModelConfig):
        super().__init__(cfg)
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size,
                                         dtype=cfg.dtype)
        self.embed_tokens.weight.requires_grad_(False)
        bg = cfg.bigram
        self.bigram = nn.Parameter(
            torch.empty(bg.buckets + 1, cfg.hidden_size, dtype=cfg.dtype),
            requires_grad=False) if bg is not None else None
        self.layers = nn.ModuleList(
            [MuneraxLayer(cfg, s) for s in cfg.layer_specs])
        self.norm = f32_vector(cfg.hidden_size)

    @property
    def lm_head(self):
        """The embedding table itself (without the input scale)."""
        return self.embed_tokens.weight

    def stack_state(self, num_slots, device) -> Dict:
        if self.bigram is None:
            return {}
        return {"prev_token": torch.zeros(num_slots, dtype=torch.long,
                                          device=device)}

    def decode_graph_capturable(self) -> bool:
        """True when no decode-step op reads device data on the host: the
        routed layers must take the fused grouped-GEMM path."""
        return all(
            not isinstance(layer.mlp, MoEMLP) or (
                self.cfg.dtype == torch.bfloat16
                and self.cfg.hidden_size % 64 == 0
                and layer.mlp.ie_local % 64 == 0)
            for layer in self.layers)

    def forward(self, input_ids, positions, kv_caches, meta,
                hidden_in=None) -> torch.Tensor:
        cfg = self.cfg
        bg = cfg.bigram
        n = len(self.layers)
        x32 = ops.bigram_embed(
            input_ids, self.embed_tokens.weight, cfg.embed_scale,
            self.bigram, bg.buckets if bg else 0, bg.mul_prev if bg else 0,
            bg.mul_cur if bg else 0,
            kv_caches[n]["prev_token"] if bg else None, meta.cu_seqlens,
            meta.state_slots, meta.seq_starts, meta.token_seq)
        h = ops.rms_norm_cast(x32, self.layers[0].norm1, cfg.rms_eps,
                              cfg.dtype)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else None
            src = layer.spec.latent.kv_from
            h = layer(x32, h, positions, kv_caches[i if src is None else src],
                      meta, nxt)
            if self.layer_hook is not None:
                self.layer_hook(i, x32)
        return x32

    # ---- weights ----------------------------------------------------------
    @torch.no_grad()
    def random_init(self, seed: int = 0):
        """Random weights of the right shapes with magnitudes that keep
        every mechanism active."""
        dev = self.norm.device
        gen = torch.Generator(device=dev).manual_seed(seed)

        def normal(p, std):
            t = torch.empty(p.shape, dtype=torch.float32, device=dev)
            t.normal_(0, std, generator=gen)
            p.copy_(t.to(p.dtype))

        def uniform(p, lo, hi):
            t = torch.empty(p.shape, dtype=torch.float32, device=dev)
            t.uniform_(lo, hi, generator=gen)
            p.copy_(t.to(p.dtype))

        for name, p in self.named_parameters():
            last = name.split(".")[-1]
            if last in ("norm", "norm1", "norm2", "kv_norm"):
                uniform(p, 0.8, 1.2)
            elif last == "sinks":
                normal(p, 0.5)
            elif "embed" in name or last == "bigram":
                normal(p, 0.5 / max(self.cfg.embed_scale, 1.0))
            else:
                normal(p, 1.0 / math.sqrt(p.shape[-1]))
        return self
