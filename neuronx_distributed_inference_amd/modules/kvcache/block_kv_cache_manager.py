"""Paged (block) KV cache for paged attention / prefix caching.

Analog of the reference's `modules/kvcache/block_kv_cache_manager.py`
(layout :40-91, gather :150-182, scatter :268-375). Layout here is
(num_blocks, block_size, Hkv/rank, D) so a block's tokens are contiguous —
the decode kernel walks the block table per sequence.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from neuronx_distributed_inference_amd import ops
from neuronx_distributed_inference_amd.parallel import state as ps


class BlockKVCacheManager(nn.Module):
    is_paged = True

    def __init__(
        self,
        num_layers: int,
        num_kv_heads: int,
        head_dim: int,
        num_blocks: int,
        block_size: int = 128,
        dtype: torch.dtype = torch.bfloat16,
        tp_degree: Optional[int] = None,
        layer_kv_shapes: Optional[List[Optional[Tuple[int, int, int]]]] = None,
        state_slots: int = 0,
        layer_kv_source: Optional[List[Optional[int]]] = None,
    ):
        """`layer_kv_shapes`: optional per-layer (kv_heads, k_head_dim,
        v_head_dim) for models whose layers differ or whose keys and values
        have different head sizes; overrides num_kv_heads/head_dim. An entry
        of None is a layer without pages of its own (a recurrent layer, or
        one that reads another layer's pages: `layer_kv_source[i]` names the
        lender and `get_cache(i)` returns its tensors); v_head_dim 0 is a
        layer whose values are channels of its key rows (latent caches): it
        gets key pages only.
        `state_slots` > 0 attaches a :class:`RecurrentStateManager` as
        ``self.state`` for models that also carry fixed-size per-sequence
        state (linear recurrences, short-convolution tails)."""
        super().__init__()
        tp = tp_degree or ps.get_tensor_model_parallel_size()
        self.num_kv_heads_per_rank = max(num_kv_heads // tp, 1)
        self.head_dim = head_dim
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.num_layers = num_layers
        self.dtype = dtype
        if layer_kv_shapes is None:
            layer_kv_shapes = [(num_kv_heads, head_dim, head_dim)] * num_layers
        assert len(layer_kv_shapes) == num_layers
        self.layer_kv_shapes = [None if sh is None else (max(sh[0] // tp, 1), sh[1], sh[2])
                                for sh in layer_kv_shapes]
        self.layer_kv_source = list(layer_kv_source or [None] * num_layers)
        for i, src in enumerate(self.layer_kv_source):
            if src is not None:
                assert self.layer_kv_shapes[i] is None and self.layer_kv_shapes[src] is not None, \
                    "a borrowing layer owns no pages and its lender does"

        def pages(sh, which):
            if sh is None or sh[which] == 0:
                return torch.zeros(0, dtype=dtype)          # placeholder: no pages
            return torch.zeros((num_blocks, block_size, sh[0], sh[which]), dtype=dtype)

        self.k_caches = nn.ParameterList(
            nn.Parameter(pages(sh, 1), requires_grad=False) for sh in self.layer_kv_shapes)
        self.v_caches = nn.ParameterList(
            nn.Parameter(pages(sh, 2), requires_grad=False) for sh in self.layer_kv_shapes)
        self.state = RecurrentStateManager(state_slots) if state_slots > 0 else None

    @property
    def has_recurrent_state(self) -> bool:
        return self.state is not None

    def estimate_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for c in (self.k_caches, self.v_caches)
                   for t in c)

    # per-forward step context set by DecoderModel (block table + slots)
    def set_step_context(self, block_table: torch.Tensor, slot_mapping: torch.Tensor):
        self._block_table = block_table
        self._slot_mapping = slot_mapping

    @property
    def block_table(self):
        return self._block_table

    @property
    def slot_mapping(self):
        return self._slot_mapping

    def get_cache(self, layer_idx: int, bucket_len=None):
        src = self.layer_kv_source[layer_idx]
        if src is not None:
            layer_idx = src
        return self.k_caches[layer_idx], self.v_caches[layer_idx]

    def update_cache(self, layer_idx: int, k_new, v_new, positions, seq_ids=None):
        """Same contract as the linear manager: k_new/v_new (B,Hkv,S,D);
        routes through the slot mapping installed by set_step_context."""
        B, Hkv, S, D = k_new.shape
        k_flat = k_new.transpose(1, 2).reshape(B * S, Hkv, D)
        v_flat = v_new.transpose(1, 2).reshape(B * S, Hkv, D)
        self.update(layer_idx, k_flat, v_flat, self._slot_mapping)

    def update(self, layer_idx: int, k_new: torch.Tensor, v_new: torch.Tensor,
               slot_mapping: torch.Tensor) -> None:
        """k_new/v_new: (N_tokens, Hkv, D); slot_mapping: (N_tokens,) flat
        slot = block_id * block_size + offset, or -1 to drop."""
        ops.block_kv_cache_update(
            self.k_caches[layer_idx].data, self.v_caches[layer_idx].data,
            k_new, v_new, slot_mapping,
        )

    def gather(self, layer_idx: int, block_table: torch.Tensor, max_len: int
               ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Contiguous (B,Hkv,S,D) K/V view for prefix-prefill paths."""
        from neuronx_distributed_inference_amd.ops import ref
        return ref.paged_gather_kv(
            self.k_caches[layer_idx].data, self.v_caches[layer_idx].data,
            block_table, max_len,
        )

    def reset(self):
        for k in self.k_caches:
            k.data.zero_()
        for v in self.v_caches:
            v.data.zero_()
        if self.state is not None:
            self.state.reset()


class RecurrentStateManager(nn.Module):
    """Fixed-size per-sequence state beside the KV cache: one fp32 tensor
    (slots, *shape) per registered key. A slot is the engine's seq_id, the
    same index that selects a linear-cache row; kernels start from zeros
    when a row's first token has position 0, so a slot that is handed to a
    new request needs no clearing."""

    def __init__(self, num_slots: int):
        super().__init__()
        self.num_slots = num_slots
        self.tensors = nn.ParameterDict()

    @staticmethod
    def _key(name: str) -> str:
        return name.replace(".", "_")

    def register(self, name: str, shape, dtype: torch.dtype = torch.float32):
        self.tensors[self._key(name)] = nn.Parameter(
            torch.zeros((self.num_slots, *shape), dtype=dtype), requires_grad=False)

    def get(self, name: str) -> torch.Tensor:
        return self.tensors[self._key(name)].data

    def estimate_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors.values())

    def snapshot(self):
        """Copies of every state tensor (for steps that must be undone, e.g.
        the warm-up runs of a graph capture on live inputs)."""
        return {k: t.data.clone() for k, t in self.tensors.items()}

    def restore(self, snap):
        for k, v in snap.items():
            self.tensors[k].data.copy_(v)

    def reset(self):
        for t in self.tensors.values():
            t.data.zero_()


def generate_slot_mapping(block_table: torch.Tensor, positions: torch.Tensor,
                          block_size: int) -> torch.Tensor:
    """In-graph slot-mapping computation (ref
    `block_kv_cache_manager.py:376-430`): positions (B,S) + per-sequence
    block table (B, max_blocks) -> flat slots (B*S,). Negative positions
    (padding) map to slot -1 (dropped by the scatter kernel)."""
    valid = positions >= 0
    pos = positions.clamp(min=0)
    blk = (pos // block_size).clamp(max=block_table.shape[1] - 1)
    off = pos % block_size
    blocks = torch.gather(block_table.long(), 1, blk.long())
    slots = blocks * block_size + off
    slots = torch.where(valid & (blocks >= 0), slots, torch.full_like(slots, -1))
    return slots.flatten()
