"""Windowed softmax attention with a log-distance score penalty.

A rotation-free attention core: positions enter only through the additive
penalty ``-r1_h * log(1 + r2_h * (i - j))`` (two learned numbers per query
head) and through the mask — a sliding window of ``window`` keys plus the
first ``keep_first`` tokens of the sequence, which stay visible (at their
true distance) however far the window has moved on. Key and value heads may
have different sizes. An optional sigmoid output gate is fused into the
kernel epilogue.

The module owns only the bias parameters and the cache access; the q/k/v/gate
projections are the caller's (so a layer can fuse them with other
projections of the same input). K/V go to the paged cache first, then one
kernel serves prompt portions, single decoded tokens and mixed batches
alike: every query carries its own position.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.ops import seqmix


class DistanceBiasWindowAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, qk_dim: int, v_dim: int,
                 scale: float, window: int, keep_first: int = 0):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.qk_dim = qk_dim
        self.v_dim = v_dim
        self.scale = float(scale)
        self.window = int(window)
        self.keep_first = int(keep_first)
        self.r1 = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32), requires_grad=False)
        self.r2 = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32), requires_grad=False)

    def kv_shape(self):
        return (self.num_kv_heads, self.qk_dim, self.v_dim)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                kv_mgr, cache_idx: int, step: seqmix.StepLayout,
                gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """q (B,S,H*Dk), k (B,S,G*Dk), v (B,S,G*Dv), gate (B,S,H*Dv) — column
        slices of a fused projection are fine. Returns (B,S,H*Dv)."""
        B, S = q.shape[0], q.shape[1]
        kc, vc = kv_mgr.get_cache(cache_idx)
        k2 = k.reshape(B * S, k.shape[-1]) if k.is_contiguous() else k.flatten(0, 1)
        v2 = v.reshape(B * S, v.shape[-1]) if v.is_contiguous() else v.flatten(0, 1)
        seqmix.paged_kv_write(kc.data, vc.data, k2, v2, kv_mgr.slot_mapping, step)
        return seqmix.window_bias_attention(
            q, kc.data, vc.data, step, kv_mgr.block_table, self.r1, self.r2,
            self.scale, self.window, self.keep_first, self.num_heads, gate=gate,
            out_dtype=q.dtype)
