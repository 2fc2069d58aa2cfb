"""The share of the engine's cache that a layer-list model owns: per layer its pages (rows indexed
through the step's page tables) and its per-slot state (one row per sequence slot).

ModelRunner calls `model.alloc_cache(num_blocks, block_size, max_num_seqs)` once and hands the result
to every forward; the scheduler's page allocator and slot pool decide which pages and rows a sequence
uses. A sequence with an empty context starts from zero state whatever its slot holds, so slots and
pages are handed on without clearing.
"""
from __future__ import annotations

from dataclasses import dataclass, field, fields
from typing import List, Optional

import torch


@dataclass
class LayerCache:
    # pages: [num_blocks * block_size, ...] rows
    latent: Optional[torch.Tensor] = None   # latent attention: [rows, kv_rank + rot_dim] (the owner's tensor)
    k: Optional[torch.Tensor] = None        # grouped-query attention: [rows, kv_heads * dim]
    v: Optional[torch.Tensor] = None        # [rows, kv_heads * vdim]
    # per-slot state, fp32
    conv1: Optional[torch.Tensor] = None    # [slots, taps - 1, width]: inputs of the layer's first input convolution
    conv2: Optional[torch.Tensor] = None    # ... of its second
    delta: Optional[torch.Tensor] = None    # delta rule: [slots, heads, dim, dim]
    mix_conv: Optional[torch.Tensor] = None  # a mixer's own short convolution: [slots, taps - 1, channels]
    ssm: Optional[torch.Tensor] = None      # state-space recurrence: [slots, heads, state, vdim]
    gla: Optional[torch.Tensor] = None      # gated linear recurrence: [slots, heads, dim, vdim]
    gru: Optional[torch.Tensor] = None      # minimal gated recurrence: [slots, width]


@dataclass
class SeqCache:
    """Pages + per-slot state of every layer (the model's share of the engine's cache)."""
    layers: List[LayerCache] = field(default_factory=list)
    block_size: int = 16

    def tensors(self):
        seen, out = set(), []
        for L in self.layers:
            for f in fields(L):
                t = getattr(L, f.name)
                if t is not None and t.data_ptr() not in seen and t.numel():
                    seen.add(t.data_ptr())
                    out.append(t)
        return out

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors())
