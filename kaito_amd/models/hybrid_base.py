"""What the engine needs from a hybrid stack, shared by the designs built
from models/mixers.py: per-layer cache allocation (K/V pages for
attention mixers, state slots for recurrent ones), cache sizing, the
residual-stream observer and the f32 logits head."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.config import ModelConfig
from ..parallel.state import get_state


def f32_vector(n):
    return nn.Parameter(torch.empty(n, dtype=torch.float32),
                        requires_grad=False)


class MixerLayerBase(nn.Module):
    """A layer holding one or more mixers; subclasses define mixers()."""

    def mixers(self):
        raise NotImplementedError

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        out: Dict[str, torch.Tensor] = {}
        for m in self.mixers():
            for k, t in m.alloc_cache(num_blocks, block_size, num_slots,
                                      device).items():
                out[type(m).__name__ + "." + k] = t
        return out

    @staticmethod
    def _view(cache, m):
        pre = type(m).__name__ + "."
        return {k[len(pre):]: t for k, t in cache.items()
                if k.startswith(pre)}


class HybridStackBase(nn.Module):
    """Engine interface of a hybrid stack. Subclasses create
    self.layers (MixerLayerBase), self.norm (f32 weight of the final
    norm, as applied), self.lm_head, and forward()."""

    # the runner hands these models state slots and the unified chunk
    # metadata, and never the rotary-model prefill fast path
    uses_state_slots = True

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        st = get_state()
        if st.tp_size != 1 or st.pp_size != 1:
            raise NotImplementedError(
                "hybrid stacks run one replica per GPU (tp = pp = 1)")
        assert cfg.layer_specs, "hybrid model needs layer_specs"
        self.cfg = cfg
        # optional observer of the residual stream after each layer
        self.layer_hook = None

    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def init_rope(self, device, max_pos: Optional[int] = None):
        """No position table: rotations, where a design has them, are
        computed from the position inside the kernels."""

    def stack_state(self, num_slots, device) -> Dict:
        """Per-sequence state that belongs to the stack rather than to a
        layer (slot-indexed tensors); handed to forward() as the entry
        after the layers' caches. Default: none."""
        return {}

    def cache_bytes(self, block_size: int):
        """(bytes per KV page, bytes per state slot) over all layers."""
        page = 0
        slot = sum(t.element_size() * t[0].numel()
                   for t in self.stack_state(1, "cpu").values())
        for layer in self.layers:
            for m in layer.mixers():
                p, s = m.cache_bytes(block_size)
                page += p
                slot += s
        return page, slot

    def alloc_caches(self, num_blocks, block_size, num_slots,
                     device) -> List[Dict]:
        return [layer.alloc_cache(num_blocks, block_size, num_slots, device)
                for layer in self.layers] \
            + [self.stack_state(num_slots, device)]

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """hidden: rows of the f32 residual stream → f32 logits."""
        h = ops.rms_norm_cast(hidden.contiguous(), self.norm,
                              self.cfg.rms_eps, self.cfg.dtype)
        return F.linear(h, self.lm_head).float()
