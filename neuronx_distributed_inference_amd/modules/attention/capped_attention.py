"""Causal GQA softmax attention without rotation, with normed projections.

Positions enter in one place only, the query temperature: the score of query
``i`` is multiplied by ``1 + coef * ln(floor((i + 1) / every) + 1)``, so
queries sharpen slowly as the context grows. Queries and keys are RMS-normed
over the WHOLE projection (all heads at once, one weight vector of that
size) before they are split into heads; the scaled score passes
``cap * tanh(score / cap)`` before the softmax. Every one of these
(temperature, cap, scale, head sizes) is a constructor parameter and can be
switched off. Key and value heads may have different sizes.

A layer may *borrow* keys and values: constructed with ``owns_kv=False`` it
has no key/value norm weight, writes nothing, and attends over the paged
cache of the layer it is pointed at (keys as that layer cached them, after
its norm) with its own queries.

The module owns the norm weights and the cache access; the q/k/v projections
are the caller's (so they can be one fused GEMM). K/V go to the paged cache
first, then one kernel serves prompt portions, single decoded tokens and
mixed batches: every query carries its own position.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.ops import seqmix


class NormedCappedAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, qk_dim: int, v_dim: int,
                 scale: float, eps: float, softcap: float = 0.0,
                 q_temp: Optional[Tuple[float, int]] = None, owns_kv: bool = True):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.qk_dim = qk_dim
        self.v_dim = v_dim
        self.scale = float(scale)
        self.eps = float(eps)
        self.softcap = float(softcap or 0.0)
        self.q_temp = None if not q_temp else (float(q_temp[0]), int(q_temp[1]))
        self.owns_kv = owns_kv
        f32 = dict(dtype=torch.float32)
        self.q_norm = nn.Parameter(torch.ones(num_heads * qk_dim, **f32), requires_grad=False)
        if owns_kv:
            self.k_norm = nn.Parameter(torch.ones(num_kv_heads * qk_dim, **f32),
                                       requires_grad=False)

    def kv_shape(self):
        """(kv_heads, key size, value size) of the pages this layer owns."""
        return (self.num_kv_heads, self.qk_dim, self.v_dim) if self.owns_kv else None

    def forward(self, q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                kv_mgr, cache_idx: int, step: seqmix.StepLayout) -> torch.Tensor:
        """q (B,S,H*Dk), k (B,S,G*Dk), v (B,S,G*Dv) — column slices of a
        fused projection are fine; k and v are None for a borrowing layer,
        whose ``cache_idx`` is the lender's. Returns (B,S,H*Dv)."""
        B, S = q.shape[0], q.shape[1]
        kc, vc = kv_mgr.get_cache(cache_idx)
        qn = seqmix.rms_norm(q, self.q_norm, self.eps, out_dtype=q.dtype)
        if self.owns_kv:
            kn = seqmix.rms_norm(k, self.k_norm, self.eps, out_dtype=k.dtype)
            seqmix.paged_kv_write(kc.data, vc.data, kn.view(B * S, -1), v.flatten(0, 1),
                                  kv_mgr.slot_mapping, step)
        return seqmix.paged_attention(
            qn, kc.data, vc.data, step, kv_mgr.block_table, self.scale, self.num_heads,
            softcap=self.softcap, q_temp=self.q_temp, out_dtype=q.dtype)
