"""Lokedra: a looped stack of parallel layers served by the paged engine.

Every layer reads one norm of the stream,  h = rms(x)·(1 + w),  and adds
both sub-layers at once:

    x ← x + s₁ ⊙ mixer(shift(h)) + s₂ ⊙ ff(h)

with per-channel layer scales s₁, s₂ and the token shift  shift(h)_t =
h_t + (h_{t−1} − h_t) ⊙ μ  in front of the mixer only (the previous
token's h is per-sequence state in every layer). The stream x is f32;
sub-layers see the norm rounded to the activation dtype. Mixers
(models/mixers.py): DiagDeltaMixer (generalized delta rule),
LatentAttention (low-rank queries, interleaved rotation with
interpolated frequencies) and a parallel pair — RotaryWindowAttention
with a chunked mask, convolved q/k, keys as values and a unit sink beside
HGRN2Mixer — summed with config weights. The feed-forward is the
engine's MoEMLP with clamped-GLU experts and softmax routing whose choice
carries a per-expert correction.

A block of layers may be repeated on shared weights (LoopSpec): every
execution ("run") of a layer keeps caches and states of its own, and from
the second pass on a pass opens by adding the embedding output back
into the stream. Output: the model's norm, then the embedding table
as the head.

The residual add of a layer is fused with the norm of the next run
(ops.scaled_residual_add_norm), so a layer receives its normed input and
is told the weight of the norm that follows.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import ModelConfig
from .hybrid_base import HybridStackBase, MixerLayerBase, f32_vector
from .hybrid_config import LayerSpec, layer_moe_config
from .mixers import (DiagDeltaMixer, HGRN2Mixer, LatentAttention,
                     RotaryWindowAttention)
from .moe import MoEMLP


def layer_runs(n_layers: int, loop) -> List[tuple]:
    """Execution order as (layer index, add the embedding output first)."""
    if loop is None:
        return [(i, False) for i in range(n_layers)]
    runs = [(i, False) for i in range(loop.start)]
    for p in range(loop.times):
        runs += [(i, p > 0 and i == loop.start)
                 for i in range(loop.start, loop.stop)]
    return runs + [(i, False) for i in range(loop.stop, n_layers)]


class LokedraLayer(MixerLayerBase):
    def __init__(self, cfg: ModelConfig, spec: LayerSpec):
        super().__init__()
        self.cfg, self.spec = cfg, spec
        h, eps, dt = cfg.hidden_size, cfg.rms_eps, cfg.dtype
        self.norm1 = f32_vector(h)          # 1 + w
        self.shift = f32_vector(h)
        self.attn = self.hgrn = self.mixer = None
        if spec.kind == "general_delta":
            self.mixer = DiagDeltaMixer(h, spec.ddelta, dt, eps)
        elif spec.kind == "latent_attention":
            self.mixer = LatentAttention(h, spec.latent, dt, eps)
        elif spec.kind == "parallel":
            self.attn = RotaryWindowAttention(h, spec.rattn, dt, eps)
            self.hgrn = HGRN2Mixer(h, spec.hgrn, dt, eps)
        else:
            raise ValueError(spec.kind)
        # layer scales with the branch weights folded in at load:
        # one vector per term of the residual sum
        self.scale_mix = f32_vector(h)
        self.scale_mix2 = f32_vector(h) if spec.kind == "parallel" else None
        self.mlp = MoEMLP(layer_moe_config(cfg, spec.moe)) \
            if spec.moe is not None else None
        self.scale_ff = f32_vector(h) if self.mlp is not None else None

    def mixers(self):
        return [m for m in (self.mixer, self.attn, self.hgrn)
                if m is not None]

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        out = super().alloc_cache(num_blocks, block_size, num_slots, device)
        out["shift"] = torch.zeros(num_slots, self.cfg.hidden_size,
                                   dtype=self.cfg.dtype, device=device)
        return out

    def slot_bytes(self) -> int:
        """State of the layer itself: the previous token's normed input."""
        return self.cfg.hidden_size * torch.empty(
            0, dtype=self.cfg.dtype).element_size()

    def forward(self, x32, h, positions, cache, meta, next_norm, x_add):
        """h = rms(x32)·norm1 in the activation dtype. Adds both
        sub-layers (and x_add, the embedding output, when the next run
        opens a loop pass) to x32 and returns the next run's normed input
        (None after the last)."""
        hs = ops.token_shift(h, self.shift, cache["shift"], meta.cu_seqlens,
                             meta.state_slots, meta.seq_starts,
                             meta.token_seq)
        if self.mixer is not None:
            terms = [(self.mixer(hs, positions,
                                 self._view(cache, self.mixer), meta),
                      self.scale_mix)]
        else:
            terms = [(self.attn(hs, positions, self._view(cache, self.attn),
                                meta), self.scale_mix),
                     (self.hgrn(hs, positions, self._view(cache, self.hgrn),
                                meta), self.scale_mix2)]
        if self.mlp is not None:
            terms.append((self.mlp(h), self.scale_ff))
        return ops.scaled_residual_add_norm(
            x32, terms, next_norm, self.cfg.rms_eps, self.cfg.dtype,
            x_add=x_add)


class LokedraForCausalLM(HybridStackBase):
    def __init__(self, cfg: ModelConfig):
        super().__init__(cfg)
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size,
                                         dtype=cfg.dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(
            [LokedraLayer(cfg, s) for s in cfg.layer_specs])
        self.norm = f32_vector(cfg.hidden_size)      # 1 + w
        self.runs = layer_runs(len(self.layers), cfg.layer_loop)
        assert self.runs, "no layer is ever run"

    @property
    def lm_head(self):
        """The embedding table itself (without the input scale)."""
        return self.embed_tokens.weight

    # every run of a layer keeps its own cache and state
    def cache_bytes(self, block_size: int):
        page = slot = 0
        for li, _ in self.runs:
            layer = self.layers[li]
            slot += layer.slot_bytes()
            for m in layer.mixers():
                p, s = m.cache_bytes(block_size)
                page += p
                slot += s
        return page, slot

    def alloc_caches(self, num_blocks, block_size, num_slots,
                     device) -> List[Dict]:
        return [self.layers[li].alloc_cache(num_blocks, block_size,
                                            num_slots, device)
                for li, _ in self.runs]

    def decode_graph_capturable(self) -> bool:
        """True when no decode-step op reads device data on the host: the
        routed layers must take the fused grouped-GEMM path."""
        return all(
            layer.mlp is None or (
                self.cfg.dtype == torch.bfloat16
                and self.cfg.hidden_size % 64 == 0
                and layer.mlp.ie_local % 64 == 0)
            for layer in self.layers)

    def forward(self, input_ids, positions, kv_caches, meta,
                hidden_in=None) -> torch.Tensor:
        cfg = self.cfg
        eps, dt = cfg.rms_eps, cfg.dtype
        x32 = self.embed_tokens(input_ids).float() * cfg.embed_scale
        x0 = x32.clone() if any(add for _, add in self.runs) else None
        h = ops.rms_norm_cast(x32, self.layers[self.runs[0][0]].norm1, eps,
                              dt)
        last = len(self.runs) - 1
        for j, (li, _) in enumerate(self.runs):
            nxt = self.runs[j + 1] if j < last else None
            next_norm = self.layers[nxt[0]].norm1 if nxt else None
            x_add = x0 if nxt and nxt[1] else None
            if self.layer_hook is not None and x_add is not None:
                # an observer sees the stream as the layer leaves it,
                # before the next pass's input is added
                self.layers[li](x32, h, positions, kv_caches[j], meta, None,
                                None)
                self.layer_hook(j, x32)
                x32 += x_add
                h = ops.rms_norm_cast(x32, next_norm, eps, dt)
                continue
            h = self.layers[li](x32, h, positions, kv_caches[j], meta,
                                next_norm, x_add)
            if self.layer_hook is not None:
                self.layer_hook(j, x32)
        return x32

    # ---- weights ----------------------------------------------------------
    @torch.no_grad()
    def random_init(self, seed: int = 0):
        """Random weights of the right shapes with magnitudes that keep
        every mechanism active (decays away from 0 and 1, gates open)."""
        dev = self.norm.device
        gen = torch.Generator(device=dev).manual_seed(seed)

        def normal(p, std, mean=0.0):
            t = torch.empty(p.shape, dtype=torch.float32, device=dev)
            t.normal_(mean, std, generator=gen)
            p.copy_(t.to(p.dtype))

        def uniform(p, lo, hi):
            t = torch.empty(p.shape, dtype=torch.float32, device=dev)
            t.uniform_(lo, hi, generator=gen)
            p.copy_(t.to(p.dtype))

        for name, p in self.named_parameters():
            last = name.split(".")[-1]
            if last in ("norm", "norm1", "out_norm", "kv_norm", "q_norm"):
                uniform(p, 0.8, 1.2)
            elif last == "shift":
                uniform(p, 0.0, 1.0)
            elif last.startswith("scale_"):
                uniform(p, 0.2, 0.6)
            elif last == "lower":
                uniform(p, 0.0, 0.9)
            elif last in ("a_bias", "f_bias", "qkv_bias", "o_bias"):
                normal(p, 0.5)
            elif last == "w0":
                normal(p, 2.0, -1.0)
            elif last == "e_score_correction_bias":
                normal(p, 0.05)
            elif last == "conv_weight":
                normal(p, 0.5)
            elif "embed" in name:
                normal(p, 0.5 / max(self.cfg.embed_scale, 1.0))
            else:
                normal(p, 1.0 / math.sqrt(p.shape[-1]))
        return self
