"""Linear attention with a recurrent state per request: a decay per head, the gated delta rule, or a state-space
recurrence whose decay depends on the token.

Per head ``S_t = decay[h] * S_(t-1) + k_t v_t^T`` and ``o_t = S_t^T q_t``: no softmax, no cache that grows with the
sequence.  What a request carries from token to token is the ``dim x vdim`` matrix ``S`` of every head, in fp32, one
slot per row of the worker's persistent batch (``AttentionMetadata.state_slots``; the model runner allocates the
tensor next to the KV cache and adds a spare slot for the padding rows of captured decode batches).  Nothing is cleared
when a slot changes owner: rows that start at position 0 take the state as zero whatever the slot holds.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
import torch.nn as nn

from ... import ops
from .attention import get_forward_context
from .linear import ColumnParallelLinear, ReplicatedLinear
from .short_conv import ShortConv, SlotState


class DecayLinearAttention(nn.Module):
    """Reads ``[q | k | v]`` from the leading columns of a fused projection (``activation``: through SiLU first),
    returns the fp32 heads ``[T, H * vdim]`` side by side."""
    state_dtype = torch.float32

    def __init__(self, num_heads: int, dim: int, vdim: int, decay: Sequence[float], layer_idx: int,
                 activation: bool = True):
        super().__init__()
        if len(decay) != num_heads:
            raise ValueError(f"layer {layer_idx}: {len(decay)} decays for {num_heads} heads")
        self.num_heads, self.dim, self.vdim = num_heads, dim, vdim
        self.layer_idx, self.activation = layer_idx, activation
        # fp32 from the configuration's doubles (the recurrence multiplies by exactly this number every token)
        self.register_buffer("decay", torch.tensor([float(d) for d in decay], dtype=torch.float32), persistent=False)
        self.state: Optional[torch.Tensor] = None

    # ---- per-request state, owned by the model runner
    def state_shape(self, num_slots: int) -> Tuple[int, int, int, int]:
        return (num_slots, self.num_heads, self.dim, self.vdim)

    def state_values_per_slot(self) -> int:
        return self.num_heads * self.dim * self.vdim

    def bind_state(self, state: Optional[torch.Tensor]) -> None:
        self.state = state

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        if md is None:                    # memory-profiling pass: no state bound
            return x.new_zeros((x.shape[0], self.num_heads * self.vdim), dtype=torch.float32)
        return ops.decay_linear_attention(x, self.num_heads, self.dim, self.vdim, self.decay, self.state,
                                          md.state_slots, md.query_start_loc, md.seq_lens, self.activation,
                                          md.max_query_len)


class GatedDeltaRule(nn.Module):
    """The gated delta rule: per value head a ``dim x vdim`` fp32 state with
    ``S <- g * S`` (one decay per key channel, by rows), ``u = b (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``, on
    unit-length q and k (q times ``dim^-0.5``), ``b = sigmoid(beta)`` and ``g = exp(-exp(a_log[h]) * softplus(dt +
    dt_bias))``.  ``heads`` value heads share ``qk_heads`` query / key heads in runs of neighbours.  The state tensors
    are ``layers.short_conv.SlotState`` objects the caller owns (one per run of the layer); ``forward`` reads
    ``[q | k | v]`` from the leading columns of ``x`` and returns the fp32 heads ``[T, heads * vdim]`` side by side."""

    def __init__(self, heads: int, qk_heads: int, dim: int, vdim: int, layer_idx: int, norm_eps: float = 1e-6):
        super().__init__()
        if heads % qk_heads:
            raise ValueError(f"layer {layer_idx}: {heads} value heads do not divide over {qk_heads} query / key heads")
        self.heads, self.qk_heads, self.dim, self.vdim = heads, qk_heads, dim, vdim
        self.layer_idx, self.norm_eps = layer_idx, float(norm_eps)
        self.a_log = nn.Parameter(torch.zeros(heads, dtype=torch.float32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(heads * dim, dtype=torch.float32), requires_grad=False)

    def per_slot_shape(self) -> Tuple[int, int, int]:
        return (self.heads, self.dim, self.vdim)

    def forward(self, x: torch.Tensor, beta: torch.Tensor, dt: torch.Tensor, state: Optional[torch.Tensor]) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        if md is None or state is None:   # memory-profiling pass: no state bound
            return x.new_zeros((x.shape[0], self.heads * self.vdim), dtype=torch.float32)
        return ops.gated_delta_rule(x, self.heads, self.qk_heads, self.dim, self.vdim, beta, dt, self.dt_bias,
                                    self.a_log, state, md.state_slots, md.query_start_loc, md.seq_lens, self.norm_eps,
                                    md.max_query_len)


class SelectiveStateSpace(nn.Module):
    """A state-space recurrence in its dual (attention-like) form: per head an ``n_state x vdim`` fp32 state with
    ``S <- exp(-exp(a_log[h]) * d) * S + d * B u^T`` and ``y = S^T C + d_skip[h] * u``, where the step size
    ``d = softplus(dt + dt_bias[h])`` comes from the token (unbounded above); ``heads`` heads share ``groups`` B / C vectors
    in runs of neighbours.  The state tensors are ``layers.short_conv.SlotState`` objects the caller owns;
    ``forward`` reads ``[u | B | C]`` from the leading columns of ``x`` and returns the fp32 heads
    ``[T, heads * vdim]`` side by side.  ``skip`` False: no ``d_skip`` term."""

    def __init__(self, heads: int, groups: int, vdim: int, n_state: int, layer_idx: int, skip: bool = True):
        super().__init__()
        if groups < 1 or heads % groups:
            raise ValueError(f"layer {layer_idx}: {heads} heads do not divide over {groups} B / C groups")
        self.heads, self.groups, self.vdim, self.n_state = heads, groups, vdim, n_state
        self.layer_idx = layer_idx
        f32 = torch.float32
        self.a_log = nn.Parameter(torch.zeros(heads, dtype=f32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(heads, dtype=f32), requires_grad=False)
        self.d_skip = nn.Parameter(torch.zeros(heads, dtype=f32), requires_grad=False) if skip else None

    @property
    def channels(self) -> int:
        """Columns ``forward`` reads: ``[u | B | C]``."""
        return self.heads * self.vdim + 2 * self.groups * self.n_state

    def per_slot_shape(self) -> Tuple[int, int, int]:
        return (self.heads, self.n_state, self.vdim)

    def forward(self, x: torch.Tensor, dt: torch.Tensor, state: Optional[torch.Tensor]) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        if md is None or state is None:   # memory-profiling pass: no state bound
            return x.new_zeros((x.shape[0], self.heads * self.vdim), dtype=torch.float32)
        return ops.selective_scan(x, dt, self.heads, self.groups, self.vdim, self.n_state, self.a_log, self.dt_bias,
                                  self.d_skip, state, md.state_slots, md.query_start_loc, md.seq_lens,
                                  md.max_query_len)


class DeltaRuleMixer(nn.Module):
    """Everything of a gated-delta-rule mixer between its normed input and its output projection: one fused projection
    ``[q | k | v | beta | decay rank | gate rank]``, the two low-rank up-projections, convolution + SiLU over
    ``[q | k | v]``, the recurrence, and the per-head RMS norm times the sigmoid gate.  ``passes``: how many times the
    layer runs in a forward pass over these weights (each run with convolution tails and a state of its own);
    ``forward`` writes ``scale * normed, gated heads`` into the columns it is given, so a caller may fuse several
    mixers' output projections."""

    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype, passes: int, scale: float):
        super().__init__()
        self.heads, self.qk_heads = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
        self.dim, self.vdim = int(m["dim"]), int(m.get("vdim") or m["dim"])
        self.decay_rank, self.gate_rank = int(m["decay_rank"]), int(m["gate_rank"])
        self.eps, self.dtype, self.out_scale = eps, dtype, float(scale)
        qs, vs = self.qk_heads * self.dim, self.heads * self.vdim
        self.channels, self.out_cols = 2 * qs + vs, vs
        self.proj = ColumnParallelLinear(width, [qs, qs, vs, self.heads, self.decay_rank, self.gate_rank], False, dtype)
        self.a2 = ReplicatedLinear(self.decay_rank, self.heads * self.dim, False, dtype)
        self.g2 = ReplicatedLinear(self.gate_rank, vs, False, dtype)
        self.conv = ShortConv([qs, qs, vs], int(m.get("conv") or 1), dtype)
        self.rule = GatedDeltaRule(self.heads, self.qk_heads, self.dim, self.vdim, layer_idx)
        self.conv_states = [SlotState((max(self.conv.taps - 1, 1), self.channels)) for _ in range(passes)]
        self.rule_states = [SlotState(self.rule.per_slot_shape(), torch.float32) for _ in range(passes)]
        self.norm = nn.Parameter(torch.zeros(self.vdim, dtype=torch.float32), requires_grad=False)

    def forward(self, h: torch.Tensor, index: int, out: torch.Tensor) -> None:
        ctx = get_forward_context()
        md = ctx.attn_metadata
        x = self.proj(h)
        c = self.channels
        dt = self.a2(x[:, c + self.heads:c + self.heads + self.decay_rank])
        gate = self.g2(x[:, c + self.heads + self.decay_rank:])
        if md is None:                    # memory-profiling pass: no state
            out.zero_()
            return
        rows = None if md.num_prefills == 0 else md.token_rows(ctx.positions)[0]
        qkv = ops.short_conv_act(x, c, self.conv.weight_t, self.conv_states[index].state, md.state_slots,
                                 md.query_start_loc, md.seq_lens, rows, ctx.positions, True, md.num_prefills > 0)
        o = self.rule(qkv, x[:, c:c + self.heads], dt, self.rule_states[index].state)
        ops.gated_rms_norm(o, self.norm, gate, self.eps, self.dtype, group=self.vdim, scale=self.out_scale, out=out)
