"""Short causal convolutions over the columns of a fused projection, with per-request state.

A layer that convolves its projections over time has to remember the last ``taps - 1`` projected rows of every
live request: a prompt may arrive in portions, and a decoded token needs its predecessors' projections.  That
state lives in one tensor per layer, ``[slots, taps - 1, channels]`` in the model dtype, indexed by the request's
row in the worker's persistent batch (``AttentionMetadata.state_slots``); the model runner allocates it next to
the KV cache.  Nothing is cleared when a row changes owner: positions before a sequence's start read as zero
because of where they are, not because of what the slot holds.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
import torch.nn as nn


class ShortConv(nn.Module):
    """``weight[channels, taps]`` for the leading ``channels`` columns of a fused projection; the checkpoint may
    hold it in pieces (one per projection), loaded into consecutive row ranges.  ``bias``: one fp32 number per
    channel, added to the convolution's sum."""

    def __init__(self, piece_sizes: Sequence[int], taps: int, dtype: torch.dtype, bias: bool = False):
        super().__init__()
        self.piece_sizes = list(piece_sizes)
        self.channels, self.taps = sum(self.piece_sizes), int(taps)
        if self.taps < 1:
            raise ValueError("a convolution needs at least one tap")
        self.weight = nn.Parameter(torch.empty(self.channels, self.taps, dtype=dtype), requires_grad=False)
        self.weight.weight_loader = self.load_piece          # type: ignore[attr-defined]
        self.bias = nn.Parameter(torch.zeros(self.channels, dtype=torch.float32), requires_grad=False) if bias else None
        self.state: Optional[torch.Tensor] = None
        self.dtype = dtype
        # what the kernels read: the same numbers tap-major, ``[taps, channels]`` (the taps of neighbouring
        # channels side by side: one 16-byte load per tap and lane); made once the checkpoint is in
        self.register_buffer("weight_t", None)

    def finalize_weights(self) -> None:
        self.weight_t = self.weight.data.t().contiguous()

    def load_piece(self, param: nn.Parameter, w: torch.Tensor, shard_id: Optional[int] = None) -> None:
        from ..utils import materialize
        w = materialize(w)
        if shard_id is None:
            assert tuple(w.shape) == tuple(param.shape), (w.shape, param.shape)
            param.data.copy_(w)
            return
        off, n = sum(self.piece_sizes[:shard_id]), self.piece_sizes[shard_id]
        assert tuple(w.shape) == (n, self.taps), (w.shape, n, self.taps)
        param.data[off:off + n].copy_(w)

    # ---- per-request state, owned by the model runner
    def state_shape(self, num_slots: int) -> Tuple[int, int, int]:
        return (num_slots, max(self.taps - 1, 1), self.channels)

    def state_values_per_slot(self) -> int:
        return max(self.taps - 1, 1) * self.channels

    def bind_state(self, state: Optional[torch.Tensor]) -> None:
        self.state = state


class SlotState:
    """One per-request state tensor, ``[slots, *per_slot]``, of a layer whose weights live elsewhere: a layer that
    runs several times in a forward pass over the same weights keeps one of these per run (the model lists them in
    ``state_layers()``; the model runner allocates and binds them like a ``ShortConv``'s own state).
    ``state_dtype`` None: the model dtype."""

    def __init__(self, per_slot: Sequence[int], state_dtype: Optional[torch.dtype] = None):
        self.per_slot = tuple(int(n) for n in per_slot)
        self.state_dtype = state_dtype
        self.state: Optional[torch.Tensor] = None

    def state_shape(self, num_slots: int) -> Tuple[int, ...]:
        return (num_slots,) + self.per_slot

    def state_values_per_slot(self) -> int:
        n = 1
        for d in self.per_slot:
            n *= d
        return n

    def bind_state(self, state: Optional[torch.Tensor]) -> None:
        self.state = state
