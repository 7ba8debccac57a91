"""Shared graph-body plumbing of the hybrid decoders (models that mix paged
attention layers with recurrent layers on an fp32 residual stream).

:class:`HybridDecoderModel` fills the engine hooks of
:class:`DecoderModel` once for all of them:

- a :class:`seqmix.StepLayout` per step (positions, state slots, valid
  counts) installed on the cache manager, and a linear block table for
  callers that bring none;
- one :class:`BlockKVCacheManager` whose per-run page shapes, lenders and
  recurrent-state tensors are collected from the layers: a layer exposes
  ``kv_shape()`` (None when it owns no pages), ``kv_source()`` (layer index
  it borrows pages from, or None) and ``state_shapes()``;
- the fp32 residual stream (embedding widened, optionally scaled).

A subclass builds its layers and may override :meth:`run_order` (layers that
repeat) and the remaining hooks.
"""

from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd.models.model_base import DecoderModel
from neuronx_distributed_inference_amd.modules.attention.attention_base import PHASE_CTE
from neuronx_distributed_inference_amd.ops import seqmix


class LayerRun:
    """One execution of a hybrid layer against its own cache/state index,
    with the engine's layer-call signature."""

    def __init__(self, layer: nn.Module, run_idx: int):
        self.layer = layer
        self.run_idx = run_idx

    def __call__(self, h, residual, cos, sin, kv_mgr, position_ids, phase,
                 attention_mask, seq_ids, **_):
        # context encoding = every row starts its sequence in this step;
        # mixers may take a whole-prompt path then
        kv_mgr.step.fresh = phase == PHASE_CTE
        return self.layer(h, kv_mgr, self.run_idx), None


class HybridDecoderModel(DecoderModel):
    embed_scale: Optional[float] = None

    def build_rotary(self, config):
        return None           # layers that rotate own their frequency tables

    def run_order(self, config) -> List[int]:
        """Layer index of every layer run, in execution order."""
        return list(range(len(self.layers)))

    def build_kv_manager(self, config) -> nn.Module:
        from neuronx_distributed_inference_amd.modules.kvcache.block_kv_cache_manager import (
            BlockKVCacheManager,
        )

        ec = config.neuron_config
        self._order = self.run_order(config)
        self._runs = [(li, LayerRun(self.layers[li], ri)) for ri, li in enumerate(self._order)]
        first_run: Dict[int, int] = {}
        for ri, li in enumerate(self._order):
            first_run.setdefault(li, ri)
        shapes, sources = [], []
        for li in self._order:
            layer = self.layers[li]
            src = layer.kv_source() if hasattr(layer, "kv_source") else None
            shapes.append(None if src is not None else layer.kv_shape())
            sources.append(None if src is None else first_run[src])
        self.max_blocks_per_seq = (ec.max_length + ec.pa_block_size - 1) // ec.pa_block_size
        num_blocks = ec.pa_num_blocks or self.max_blocks_per_seq * ec.kv_cache_batch_size
        mgr = BlockKVCacheManager(
            num_layers=len(self._order), num_kv_heads=1, head_dim=1,
            num_blocks=num_blocks, block_size=ec.pa_block_size, dtype=ec.torch_dtype,
            tp_degree=1, layer_kv_shapes=shapes, layer_kv_source=sources,
            state_slots=ec.kv_cache_batch_size,
        )
        for ri, li in enumerate(self._order):
            for name, shape in self.layers[li].state_shapes().items():
                mgr.state.register(f"run{ri}.{name}", shape)
        return mgr

    # -- engine hooks ---------------------------------------------------
    def begin_step(self, position_ids, seq_ids, block_table):
        B = position_ids.shape[0]
        if seq_ids is None:
            seq_ids = torch.arange(B, device=position_ids.device)
        self.kv_mgr.step = seqmix.StepLayout(position_ids, seq_ids)
        if block_table is None:
            # callers without a page table (plain generate loops) get the
            # linear layout: slot s owns pages [s*M, (s+1)*M)
            M = self.max_blocks_per_seq
            if self.kv_mgr.num_blocks < self.kv_mgr.state.num_slots * M:
                raise RuntimeError(
                    "the page pool is smaller than slots x max_length: pass a block_table")
            sid = seq_ids.long().view(B, 1)
            block_table = torch.where(
                sid >= 0,
                sid * M + torch.arange(M, device=position_ids.device).view(1, M),
                torch.full_like(sid, -1))     # pad rows own no pages
        return block_table

    def prepare_hidden(self, h):
        if self.embed_scale is not None:
            return seqmix.scaled_embedding(h, self.embed_scale)
        return h.float()

    def layer_runs(self):
        return self._runs

    def before_layer_run(self, run_idx, h, h_embed):
        if run_idx == 0:
            return h.clone() if h is h_embed and h.dtype == torch.float32 else h
        return h
