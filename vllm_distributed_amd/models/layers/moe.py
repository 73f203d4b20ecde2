"""Sparse mixture-of-experts MLP (Qwen3-MoE routing).

Two sharding modes over the TP group:

* tensor-sharded experts (default, what the reference's TP=2 deployment of
  Qwen3-Coder-480B-A35B uses - ``.env.server:11`` has no expert-parallel flag):
  every rank holds all experts with ``intermediate/tp`` columns;
* expert parallel (``enable_expert_parallel``): every rank holds ``E/tp`` whole
  experts and only computes the tokens routed to them.

Either way partial outputs are summed with one all-reduce.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ..utils import materialize
import torch.nn.functional as F

from ... import envs, ops
from ...parallel.state import (get_tensor_model_parallel_rank,
                               get_tensor_model_parallel_world_size,
                               tensor_model_parallel_all_reduce)
from .linear import (ReplicatedLinear, _fill_scalar, active_quant, awq_to_native, divide, fp4_layout_ok,
                     nvfp4_dequantize, w4_layout_ok)


class ExpertRows:
    """A sparse block's output before the weighted sum over each token's experts: rows ``y`` in
    expert-sorted order plus the routing tables.  An ``RMSNorm`` called with a residual sums, adds and
    normalises in one launch; everybody else asks for ``materialize()``."""
    __slots__ = ("y", "topw", "topi", "inv", "expert_start", "local")

    def __init__(self, y, topw, topi, inv, expert_start, local):
        self.y, self.topw, self.topi, self.inv, self.expert_start, self.local = y, topw, topi, inv, expert_start, local

    @property
    def shape(self):
        return (self.topi.shape[0], self.y.shape[1])

    def materialize(self) -> torch.Tensor:
        return ops.moe_combine(self.y, self.topw, self.topi, self.inv, self.expert_start, self.local)

    def add_rms_norm(self, residual: torch.Tensor, weight: torch.Tensor, eps: float):
        return ops.moe_combine_add_rms_norm(self.y, self.topw, self.topi, self.inv, self.expert_start, self.local,
                                            residual, weight, eps)


class FusedMoE(nn.Module):
    def __init__(self, hidden: int, inter: int, num_experts: int, top_k: int,
                 renormalize: bool, dtype: torch.dtype, expert_parallel: bool = False,
                 allocate_experts: bool = True):
        # allocate_experts = False: a subclass lays out its own (dense) expert tensors
        super().__init__()
        self.tp = get_tensor_model_parallel_world_size()
        self.tp_rank = get_tensor_model_parallel_rank()
        self.num_experts, self.top_k, self.renormalize = num_experts, top_k, renormalize
        self.expert_parallel = expert_parallel and self.tp > 1
        if self.expert_parallel:
            self.local_experts = divide(num_experts, self.tp)
            self.expert_start = self.tp_rank * self.local_experts
            self.inter_local = inter
        else:
            self.local_experts, self.expert_start = num_experts, 0
            self.inter_local = divide(inter, self.tp)
        self.inter = inter
        self.hidden, self.dtype = hidden, dtype
        self.gate = ReplicatedLinear(hidden, num_experts, False, dtype, quant=False)   # router stays dense
        self.quant = active_quant()
        if self.quant is not None and self.quant.method not in ("awq", "nvfp4"):
            self.quant = None           # fp8 covers the dense linears; experts stay in the model dtype
        E, I = self.local_experts, self.inter_local
        self.register_buffer("qw13", None)
        self.register_buffer("sz13", None)
        self.register_buffer("qw2", None)
        self.register_buffer("sz2", None)
        self.register_buffer("alpha13", None)
        self.register_buffer("alpha2", None)

        def param(*shape, dt=dtype, out_dim=0, pack=1, in_div=1, loader=None):
            p = nn.Parameter(torch.empty(*shape, dtype=dt), requires_grad=False)
            p.out_dim, p.pack, p.in_div, p.weight_loader = out_dim, pack, in_div, loader
            return p
        if not allocate_experts:
            return
        if self.quant is None:
            self.w13 = param(E, 2 * I, hidden, loader=self._load_w13)
            self.w2 = param(E, hidden, I, loader=self._load_w2)
        elif self.quant.method == "nvfp4":
            assert hidden % 16 == 0 and I % 16 == 0, f"NVFP4 expert shard [{I} x {hidden}] splits a 16-column block"
            u8, f8, f32 = torch.uint8, torch.float8_e4m3fn, torch.float32
            self.w13_weight_packed = param(E, 2 * I, hidden // 2, dt=u8, in_div=2, loader=self._load_w13)
            self.w13_weight_block_scale = param(E, 2 * I, hidden // 16, dt=f8, in_div=16, loader=self._load_w13)
            self.w13_weight_alpha = param(E, 2 * I, dt=f32, loader=self._load_w13)
            self.w2_weight_packed = param(E, hidden, I // 2, dt=u8, in_div=2, loader=self._load_w2)
            self.w2_weight_block_scale = param(E, hidden, I // 16, dt=f8, in_div=16, loader=self._load_w2)
            self.w2_weight_alpha = param(E, hidden, dt=f32, loader=self._load_w2)
            self.w13_weight_alpha.per_shard_scalar = self.w2_weight_alpha.per_shard_scalar = True
        else:
            g, pk = self.quant.group_size, self.quant.pack
            assert hidden % g == 0 and I % g == 0, \
                f"expert shard [{I} x {hidden}] does not align with quantisation groups of {g}"
            i32 = torch.int32
            self.w13_qweight = param(E, hidden, 2 * I // pk, dt=i32, out_dim=1, pack=pk, loader=self._load_w13)
            self.w13_qzeros = param(E, hidden // g, 2 * I // pk, dt=i32, out_dim=1, pack=pk, in_div=g,
                                    loader=self._load_w13)
            self.w13_scales = param(E, hidden // g, 2 * I, out_dim=1, in_div=g, loader=self._load_w13)
            self.w2_qweight = param(E, I, hidden // pk, dt=i32, out_dim=1, pack=pk, loader=self._load_w2)
            self.w2_qzeros = param(E, I // g, hidden // pk, dt=i32, out_dim=1, pack=pk, in_div=g,
                                   loader=self._load_w2)
            self.w2_scales = param(E, I // g, hidden, out_dim=1, in_div=g, loader=self._load_w2)

    def _local_index(self, expert_id: int) -> Optional[int]:
        e = expert_id - self.expert_start
        return e if 0 <= e < self.local_experts else None

    def _load_w13(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        expert_id, which = shard_id          # which: 0 = gate, 1 = up
        e = self._local_index(expert_id)
        if e is None:
            return
        od, pack = param.out_dim, param.pack
        n = self.inter_local // pack
        if getattr(param, "per_shard_scalar", False):
            return _fill_scalar(param.data[e].narrow(0, which * n, n), w)
        if not self.expert_parallel:
            w = w.narrow(od, self.tp_rank * n, n)
        param.data[e].narrow(od, which * n, n).copy_(materialize(w))

    def _load_w2(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        expert_id, _ = shard_id
        e = self._local_index(expert_id)
        if e is None:
            return
        if getattr(param, "per_shard_scalar", False):
            return _fill_scalar(param.data[e], w)
        if not self.expert_parallel:
            n = self.inter_local // param.in_div
            w = w.narrow(1 - param.out_dim, self.tp_rank * n, n)
        param.data[e].copy_(materialize(w))

    def finalize_weights(self) -> None:
        """Repack the experts' AWQ shards into the 4-bit kernel layout (or
        dequantise them when a shard shape does not tile)."""
        if self.quant is None or self.qw13 is not None:
            return
        E, I, H, g = self.local_experts, self.inter_local, self.hidden, self.quant.group_size
        if self.quant.method == "nvfp4":
            return self._finalize_nvfp4()
        native = w4_layout_ok(H, 2 * I, g) and w4_layout_ok(I, H, g)
        parts = {"13": [], "2": []}
        for key in ("13", "2"):
            qweight = getattr(self, f"w{key}_qweight").data
            qzeros = getattr(self, f"w{key}_qzeros").data
            scales = getattr(self, f"w{key}_scales").data
            for e in range(E):
                if native:
                    parts[key].append(awq_to_native(qweight[e], qzeros[e], scales[e], self.dtype))
                else:
                    from ..loader import awq_dequantize
                    parts[key].append(awq_dequantize(qweight[e], qzeros[e], scales[e], self.dtype))
            delattr(self, f"w{key}_qweight")
            delattr(self, f"w{key}_qzeros")
            delattr(self, f"w{key}_scales")
        if native:
            self.qw13 = torch.stack([p[0] for p in parts["13"]])
            self.sz13 = torch.stack([p[1] for p in parts["13"]])
            self.qw2 = torch.stack([p[0] for p in parts["2"]])
            self.sz2 = torch.stack([p[1] for p in parts["2"]])
            ops.w4_reserve_scratch(2 * I * H, self.qw13.device, self.dtype)
        else:
            self.quant = None
            self.w13 = nn.Parameter(torch.stack(parts["13"]), requires_grad=False)
            self.w2 = nn.Parameter(torch.stack(parts["2"]), requires_grad=False)

    def _finalize_nvfp4(self) -> None:
        from ...ops import quant
        E, I, H = self.local_experts, self.inter_local, self.hidden
        native = fp4_layout_ok(H, 2 * I) and fp4_layout_ok(I, H)
        out = {}
        for key in ("13", "2"):
            packed = getattr(self, f"w{key}_weight_packed").data
            bs = getattr(self, f"w{key}_weight_block_scale").data
            alpha = getattr(self, f"w{key}_weight_alpha").data
            for name in ("weight_packed", "weight_block_scale", "weight_alpha"):
                delattr(self, f"w{key}_{name}")
            if native:
                parts = [quant.pack_fp4(packed[e], bs[e]) for e in range(E)]
                out[key] = (torch.stack([p[0] for p in parts]), torch.stack([p[1] for p in parts]), alpha.contiguous())
            else:
                out[key] = torch.stack([nvfp4_dequantize(packed[e], bs[e], alpha[e], self.dtype) for e in range(E)])
        if native:
            self.qw13, self.sz13, self.alpha13 = out["13"]
            self.qw2, self.sz2, self.alpha2 = out["2"]
            ops.w4_reserve_scratch(2 * I * H, self.qw13.device, self.dtype)
        else:
            self.quant = None
            self.w13 = nn.Parameter(out["13"], requires_grad=False)
            self.w2 = nn.Parameter(out["2"], requires_grad=False)

    def _expert_mlp(self, e: int, x: torch.Tensor) -> torch.Tensor:
        if self.alpha13 is not None:
            h = ops.fp4_linear(x, self.qw13[e], self.sz13[e], self.alpha13[e])
            return ops.fp4_linear(ops.silu_and_mul(h), self.qw2[e], self.sz2[e], self.alpha2[e])
        if self.qw13 is not None:
            h = ops.w4a16_linear(x, self.qw13[e], self.sz13[e])
            return ops.w4a16_linear(ops.silu_and_mul(h), self.qw2[e], self.sz2[e])
        return F.linear(ops.silu_and_mul(F.linear(x, self.w13[e])), self.w2[e])

    def _grouped_tile_rows(self, x: torch.Tensor) -> int:
        """Row-tile size for the grouped HIP GEMMs, or 0 to use the per-expert
        library GEMMs (large prefill batches, where each expert has hundreds of
        rows and hipBLASLt is compute-efficient; that path syncs with the host,
        so it is never taken while a hipGraph is being captured)."""
        if not (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and ops.hip_available()):
            return 0
        if self.quant is None and (self.w13.shape[2] % 128 or self.w2.shape[2] % 128 or self.w13.shape[1] % 16):
            return 0
        cap = 64 if self.qw13 is not None else 128
        avg = x.shape[0] * self.top_k / max(1, self.num_experts)
        if avg > envs.VDAMD_MOE_GROUPED_MAX_ROWS * cap / 64 and not torch.cuda.is_current_stream_capturing():
            return 0
        for rows in (16, 32, 64, 128):
            if avg <= rows or rows == cap:
                return rows
        return cap

    def _forward_grouped(self, x: torch.Tensor, topw: torch.Tensor, topi: torch.Tensor, tile_rows: int,
                         ) -> torch.Tensor:
        """Experts as two grouped GEMMs over expert-sorted rows: no host sync,
        every expert's weights stream from HBM once per step."""
        t, k = topi.shape
        order, tiles = ops.moe_align(topi, self.num_experts, tile_rows, self.expert_start,
                                     self.local_experts if self.expert_parallel else -1)
        xs = x.index_select(0, order // k)
        if self.qw13 is not None:
            h = ops.grouped_linear(xs, tiles, tile_rows, qw=self.qw13, sz=self.sz13, alpha=self.alpha13)
            a = ops.silu_and_mul(h)
            y = ops.grouped_linear(a, tiles, tile_rows, qw=self.qw2, sz=self.sz2, alpha=self.alpha2)
        else:
            h = ops.grouped_linear(xs, tiles, tile_rows, weight=self.w13)
            a = ops.silu_and_mul(h)
            y = ops.grouped_linear(a, tiles, tile_rows, weight=self.w2)
        w_sorted = topw.reshape(-1)[order]
        if self.expert_parallel:        # rows of experts held elsewhere were never written
            local = (topi.reshape(-1)[order] >= self.expert_start) & \
                    (topi.reshape(-1)[order] < self.expert_start + self.local_experts)
            y = torch.where(local.unsqueeze(1), y, torch.zeros_like(y))
        y = y * w_sorted.unsqueeze(1)
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        return y.index_select(0, inv).view(t, k, -1).sum(dim=1)      # fixed order: deterministic

    def _experts_grouped(self, xs: torch.Tensor, tiles: torch.Tensor, tile_rows: int) -> torch.Tensor:
        if self.qw13 is not None:
            h = ops.grouped_linear(xs, tiles, tile_rows, qw=self.qw13, sz=self.sz13, alpha=self.alpha13)
            return ops.grouped_linear(h, tiles, tile_rows, qw=self.qw2, sz=self.sz2, alpha=self.alpha2,
                                      silu_mul=True)
        h = ops.grouped_linear(xs, tiles, tile_rows, weight=self.w13)
        return ops.grouped_linear(ops.silu_and_mul(h), tiles, tile_rows, weight=self.w2)

    def _forward_fused_routing(self, x: torch.Tensor, logits: torch.Tensor, tile_rows: int, deferred: bool = False):
        """Routing, expert GEMMs and the weighted sum in eight launches (router
        GEMM included): top-k, slot sort + tile table and the combine are one HIP
        kernel each.  ``deferred`` (decode-sized batches): the weighted sum is left to the add + RMSNorm
        that follows (``ExpertRows``)."""
        local = self.local_experts if self.expert_parallel else -1
        if ops.moe_route_small_ok(logits, x):
            # decode-sized batch: top-k, slot sort, tile table and the row gather are one launch
            topw, topi, inv, tiles, xs = ops.moe_route_small(logits, x, self.top_k, self.renormalize, tile_rows,
                                                             self.expert_start, local)
            y = self._experts_grouped(xs, tiles, tile_rows)
            if deferred:
                return ExpertRows(y, topw, topi, inv, self.expert_start, local)
            return ops.moe_combine(y, topw, topi, inv, self.expert_start, local)
        topw, topi = ops.moe_topk(logits, self.top_k, self.renormalize)
        src_row, inv, tiles = ops.moe_align_fused(topi, self.num_experts, tile_rows, self.expert_start, local)
        y = self._experts_grouped(x.index_select(0, src_row), tiles, tile_rows)
        return ops.moe_combine(y, topw, topi, inv, self.expert_start, local)

    # True in subclasses that override ``route``: the fused top-k kernel (softmax routing) is skipped
    custom_routing = False

    def router_logits(self, x: torch.Tensor) -> torch.Tensor:
        """``[T, E]`` scores of the router (families that keep the router in fp32 override this)."""
        return self.gate(x)

    def route(self, logits: torch.Tensor):
        """Router logits ``[T, E]`` (fp32) -> (weights ``[T, k]`` fp32, expert ids ``[T, k]``)."""
        probs = torch.softmax(logits, dim=-1)
        topw, topi = probs.topk(self.top_k, dim=-1)
        if self.renormalize:
            topw = topw / topw.sum(-1, keepdim=True)
        return topw, topi

    def forward(self, x: torch.Tensor, reduce: bool = True, staged: bool = False, deferred: bool = False):
        # `deferred`: the caller feeds the result to an add + RMSNorm and accepts ``ExpertRows``
        # `staged` (write the partial sums where the next direct all-reduce reads) is a hint only
        tile_rows = self._grouped_tile_rows(x)
        logits = None
        if (tile_rows and not self.custom_routing and self.gate.bias is None
                and getattr(self.gate, "lora", None) is None and self.num_experts <= 512 and self.top_k <= 16):
            # decode: the routing kernel adds up the router GEMM's K-split partial sums itself
            logits = ops.router_logit_partials(x, self.gate.weight)
            if logits is not None:
                # unsharded experts only: a sharded block's sum still has to cross the TP group
                defer = deferred and self.tp == 1 and envs.VDAMD_FUSED_REDUCE_NORM
                out = self._forward_fused_routing(x, logits, tile_rows, defer)
                if reduce and self.tp > 1:
                    out = tensor_model_parallel_all_reduce(out)
                return out
        logits = self.router_logits(x)
        if (tile_rows and x.dim() == 2 and not self.custom_routing
                and ops.moe_route_fused_ok(logits, self.num_experts, self.top_k)):
            out = self._forward_fused_routing(x, logits, tile_rows)
            if reduce and self.tp > 1:
                out = tensor_model_parallel_all_reduce(out)
            return out
        topw, topi = self.route(logits.float())
        topw = topw.to(x.dtype)
        if tile_rows:
            out = self._forward_grouped(x, topw, topi, tile_rows)
            if reduce and self.tp > 1:
                out = tensor_model_parallel_all_reduce(out)
            return out
        out = torch.zeros_like(x)
        # group token-slots by expert: one sort, then contiguous segments
        flat_e = topi.reshape(-1)
        order = flat_e.argsort(stable=True)
        counts = torch.bincount(flat_e, minlength=self.num_experts).tolist()
        tok = (order // self.top_k)
        wts = topw.reshape(-1)[order]
        start = 0
        for eid, n in enumerate(counts):
            if n == 0:
                continue
            seg = slice(start, start + n)
            start += n
            e = self._local_index(eid)
            if e is None:
                continue
            rows = tok[seg]
            h = self._expert_mlp(e, x.index_select(0, rows))
            out.index_add_(0, rows, h * wts[seg].unsqueeze(1))
        if reduce and self.tp > 1:
            out = tensor_model_parallel_all_reduce(out)
        return out


def _ceil128(n: int) -> int:
    return (n + 127) // 128 * 128


class ClampedGluMLP(nn.Module):
    """One feed-forward of the clamped GLU form, ``down(g sigmoid(alpha g) (u + 1))`` with ``g = min(gate(x),
    limit)`` and ``u = clamp(up(x), -limit, limit)``, gate and up as one fused projection; no biases."""

    def __init__(self, hidden: int, inter: int, limit: float, alpha: float, dtype: torch.dtype):
        super().__init__()
        self.inter, self.limit, self.alpha = inter, float(limit), float(alpha)
        self.w13 = nn.Parameter(torch.empty(2 * inter, hidden, dtype=dtype), requires_grad=False)
        self.w2 = nn.Parameter(torch.empty(hidden, inter, dtype=dtype), requires_grad=False)
        self.w13.weight_loader = self._load_w13

    def _load_w13(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        param.data.narrow(0, int(shard_id) * self.inter, self.inter).copy_(materialize(w))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(ops.clamped_glu(ops.linear(x, self.w13), self.limit, self.alpha), self.w2)


class GroupedIdentityMoE(FusedMoE):
    """Routed experts of the clamped GLU form behind a softmax router with a per-output correction that only steers
    the choice, expert groups of neighbours (a group scores as its best member; only the best ``keep_groups`` groups
    stay eligible, the others count as minus infinity), renormalised weights, and ``identity`` trailing router
    outputs that stand for experts whose output is their input; plus an optional always-on shared expert scaled by
    ``sigmoid(shared_gate . x)``, one number per token.

    The router is fp32 (weights and product); the choice is made on ``softmax + correction``, the weights are the
    chosen outputs' softmax values over their sum.  On the GPU in 16-bit types the experts run as two grouped GEMMs
    over expert-sorted rows with their reduction dimensions zero-padded to the kernels' 128-deep tiles: the identity
    outputs are routed like experts held by nobody (no rows, no weights) and their share ``x * sum of their weights``
    is added at the end.  Elsewhere (fp32, CPU) the experts run one after the other on the library GEMM."""
    custom_routing = True

    def __init__(self, hidden: int, inter: int, num_experts: int, identity: int, top_k: int, limit: float,
                 dtype: torch.dtype, groups: int = 1, keep_groups: int = 1, alpha: float = 1.702,
                 shared_inter: int = 0, shared_limit: Optional[float] = None):
        outputs = num_experts + identity
        super().__init__(hidden, inter, outputs, top_k, True, dtype, expert_parallel=False, allocate_experts=False)
        if self.tp > 1:
            raise NotImplementedError("GroupedIdentityMoE runs unsharded")
        if groups < 1 or outputs % groups or not 1 <= keep_groups <= groups:
            raise ValueError(f"{outputs} router outputs do not form {groups} equal groups of which {keep_groups} are kept")
        if top_k > outputs:
            raise ValueError(f"top {top_k} of {outputs} router outputs")
        self.quant = None
        self.real_experts, self.identity = num_experts, identity
        self.local_experts, self.expert_start = num_experts, 0      # the identity outputs have no weights
        self.groups, self.keep_groups = groups, keep_groups
        self.limit, self.alpha = float(limit), float(alpha)
        # (router weights in the model dtype: what a 16-bit checkpoint holds is exact there, and the product is
        # formed with fp32 accumulators kept as the result)
        self.gate = ReplicatedLinear(hidden, outputs, False, dtype, quant=False)
        self.gate.e_score_correction_bias = nn.Parameter(torch.zeros(outputs, dtype=torch.float32), requires_grad=False)
        self.h_pad, self.i_pad = _ceil128(hidden), _ceil128(inter)
        E = num_experts
        # [gate rows ; up rows] (each padded to i_pad rows) x (reduction padded to h_pad); [hidden, i_pad]
        self.w13 = nn.Parameter(torch.zeros(E, 2 * self.i_pad, self.h_pad, dtype=dtype), requires_grad=False)
        self.w2 = nn.Parameter(torch.zeros(E, hidden, self.i_pad, dtype=dtype), requires_grad=False)
        self.w13.weight_loader = self._load_w13
        self.w2.weight_loader = self._load_w2
        self.shared = ClampedGluMLP(hidden, shared_inter, self.limit if shared_limit is None else shared_limit,
                                    alpha, dtype) if shared_inter else None
        self.shared_gate = ReplicatedLinear(hidden, 1, False, dtype, quant=False) if shared_inter else None

    # ------------------------------------------------------------------ loading
    def _load_w13(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        e, which = shard_id                  # which: 0 = gate, 1 = up
        dst = param.data[e, which * self.i_pad:(which + 1) * self.i_pad]
        dst.zero_()                          # (the padding included: the loader poisons fresh parameters)
        dst[:self.inter, :self.hidden].copy_(materialize(w))

    def _load_w2(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        e, _ = shard_id
        param.data[e].zero_()
        param.data[e, :, :self.inter].copy_(materialize(w))

    # ------------------------------------------------------------------ routing
    def router_logits(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear_f32(x, self.gate.weight)

    def route(self, logits: torch.Tensor):
        scores = torch.softmax(logits.float(), dim=-1)
        choice = scores + self.gate.e_score_correction_bias
        if self.groups > 1 and self.keep_groups < self.groups:
            per_group = choice.view(-1, self.groups, self.num_experts // self.groups).amax(-1)
            best = per_group.topk(self.keep_groups, dim=-1).indices
            keep = torch.zeros_like(per_group, dtype=torch.bool).scatter_(1, best, True)
            keep = keep.unsqueeze(-1).expand(-1, self.groups, self.num_experts // self.groups).reshape(choice.shape)
            choice = choice.masked_fill(~keep, float("-inf"))
        topi = choice.topk(self.top_k, dim=-1).indices
        topw = scores.gather(1, topi)
        return topw / (topw.sum(-1, keepdim=True) + 1e-20), topi

    # ------------------------------------------------------------------ compute
    def _pad(self, x: torch.Tensor) -> torch.Tensor:
        return x if self.h_pad == self.hidden else F.pad(x, (0, self.h_pad - self.hidden))

    def _expert_mlp(self, e: int, x: torch.Tensor) -> torch.Tensor:
        h = F.linear(self._pad(x), self.w13[e])
        return F.linear(ops.clamped_glu(h, self.limit, self.alpha), self.w2[e])

    def _grouped_tile_rows(self, x: torch.Tensor) -> int:
        # (the grouped GEMMs write whole 16-column tiles: the down projection's output width is `hidden`)
        if self.num_experts > 512 or self.top_k > 16 or self.groups > 64 or x.dim() != 2 or self.hidden % 16:
            return 0
        return super()._grouped_tile_rows(x)

    def decode_capturable(self, dtype: torch.dtype) -> bool:
        """Whether a decode step of this block runs without a host synchronisation (the grouped path)."""
        return (dtype in (torch.bfloat16, torch.float16) and self.hidden % 16 == 0 and self.num_experts <= 512
                and self.top_k <= 16 and self.groups <= 64)

    def forward(self, x: torch.Tensor, reduce: bool = True, staged: bool = False, deferred: bool = False):
        logits = self.router_logits(x)
        tile_rows = self._grouped_tile_rows(x)
        if tile_rows:
            grouped = self.groups if self.keep_groups < self.groups else 1
            topw, topi = ops.moe_topk_grouped(logits, self.gate.e_score_correction_bias, self.top_k, grouped,
                                              self.keep_groups if grouped > 1 else 1, False, False, True, 1.0)
            src_row, inv, tiles = ops.moe_align_fused(topi, self.num_experts, tile_rows, 0, self.real_experts)
            xs = self._pad(x).index_select(0, src_row)
            h = ops.grouped_linear(xs, tiles, tile_rows, weight=self.w13)
            y = ops.grouped_linear(ops.clamped_glu(h, self.limit, self.alpha), tiles, tile_rows, weight=self.w2)
            out = ops.moe_combine(y, topw, topi, inv, 0, self.real_experts)
        else:
            topw, topi = self.route(logits)
            acc = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            flat_e = topi.reshape(-1)
            order = flat_e.argsort(stable=True)
            counts = torch.bincount(flat_e, minlength=self.num_experts).tolist()
            tok = order // self.top_k
            wts = topw.reshape(-1)[order]
            start = 0
            for eid, n in enumerate(counts[:self.real_experts]):
                if n:
                    seg = slice(start, start + n)
                    rows = tok[seg]
                    acc.index_add_(0, rows, self._expert_mlp(eid, x.index_select(0, rows)).float() * wts[seg].unsqueeze(1))
                start += n
            out = acc.to(x.dtype)
        if not self.identity and self.shared is None:
            return out
        shared = gate = None
        if self.shared is not None:
            shared, gate = self.shared(x), self.shared_gate(x)
        return ops.expert_epilogue(out, x, topw if self.identity else None, topi if self.identity else None,
                                   self.real_experts, shared, gate)


class BiasedTopKMoE(FusedMoE):
    """Routed experts of the plain form ``down(act(up(x)))`` (no gate projection, no biases) behind a router with a
    bias: the ``top_k`` largest of ``router(x) + bias`` are chosen and weighted by the softmax over just those.

    The router is fp32 (product and bias).  On the GPU in 16-bit types the experts run as two grouped GEMMs over
    expert-sorted rows, their reduction dimensions zero-padded to the kernels' 128-deep tiles; elsewhere (fp32, CPU)
    one after the other on the library GEMM.  ``activation``: ``"gelu"`` (exact) or ``"gelu_tanh"``."""
    custom_routing = True

    def __init__(self, hidden: int, inter: int, num_experts: int, top_k: int, dtype: torch.dtype,
                 activation: str = "gelu"):
        super().__init__(hidden, inter, num_experts, top_k, True, dtype, expert_parallel=False, allocate_experts=False)
        if self.tp > 1:
            raise NotImplementedError("BiasedTopKMoE runs unsharded")
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top {top_k} of {num_experts} experts")
        if activation not in ("gelu", "gelu_tanh"):
            raise ValueError(f"unsupported expert activation {activation!r}")
        self.quant = None
        self.tanh = activation == "gelu_tanh"
        self.gate = ReplicatedLinear(hidden, num_experts, False, dtype, quant=False)
        self.gate_bias = nn.Parameter(torch.zeros(num_experts, dtype=torch.float32), requires_grad=False)
        self.h_pad, self.i_pad = _ceil128(hidden), _ceil128(inter)
        self.w1 = nn.Parameter(torch.zeros(num_experts, self.i_pad, self.h_pad, dtype=dtype), requires_grad=False)
        self.w2 = nn.Parameter(torch.zeros(num_experts, hidden, self.i_pad, dtype=dtype), requires_grad=False)
        self.w1.weight_loader = self._load_w1
        self.w2.weight_loader = self._load_w2

    def _load_w1(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        param.data[int(shard_id)].zero_()          # (the padding included: the loader poisons fresh parameters)
        param.data[int(shard_id), :self.inter, :self.hidden].copy_(materialize(w))

    def _load_w2(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        param.data[int(shard_id)].zero_()
        param.data[int(shard_id), :, :self.inter].copy_(materialize(w))

    def router_logits(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear_f32(x, self.gate.weight) + self.gate_bias

    def route(self, logits: torch.Tensor):
        val, topi = logits.float().topk(self.top_k, dim=-1)
        return torch.softmax(val, dim=-1), topi

    def _pad(self, x: torch.Tensor) -> torch.Tensor:
        return x if self.h_pad == self.hidden else F.pad(x, (0, self.h_pad - self.hidden))

    def _expert_mlp(self, e: int, x: torch.Tensor) -> torch.Tensor:
        return F.linear(ops.gelu(F.linear(self._pad(x), self.w1[e]), self.tanh), self.w2[e])

    def _grouped_tile_rows(self, x: torch.Tensor) -> int:
        if not (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and x.dim() == 2 and ops.hip_available()):
            return 0
        if self.num_experts > 512 or self.top_k > 16 or self.hidden % 16:
            return 0
        avg = x.shape[0] * self.top_k / max(1, self.num_experts)
        if avg > envs.VDAMD_MOE_GROUPED_MAX_ROWS * 2 and not torch.cuda.is_current_stream_capturing():
            return 0
        for rows in (16, 32, 64, 128):
            if avg <= rows:
                return rows
        return 128

    def decode_capturable(self, dtype: torch.dtype) -> bool:
        """Whether a decode step of this block runs without a host synchronisation (the grouped path)."""
        return (dtype in (torch.bfloat16, torch.float16) and self.hidden % 16 == 0 and self.num_experts <= 512
                and self.top_k <= 16)

    def forward(self, x: torch.Tensor, reduce: bool = True, staged: bool = False, deferred: bool = False):
        logits = self.router_logits(x)
        tile_rows = self._grouped_tile_rows(x)
        if tile_rows:
            # (softmax over every output, the largest kept and renormalised: the softmax over the kept ones)
            topw, topi = ops.moe_topk(logits, self.top_k, True)
            src_row, inv, tiles = ops.moe_align_fused(topi, self.num_experts, tile_rows, 0, -1)
            xs = self._pad(x).index_select(0, src_row)
            h = ops.grouped_linear(xs, tiles, tile_rows, weight=self.w1)
            y = ops.grouped_linear(ops.gelu(h, self.tanh), tiles, tile_rows, weight=self.w2)
            return ops.moe_combine(y, topw, topi, inv, 0, -1)
        topw, topi = self.route(logits)
        acc = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        flat_e = topi.reshape(-1)
        order = flat_e.argsort(stable=True)
        counts = torch.bincount(flat_e, minlength=self.num_experts).tolist()
        tok = order // self.top_k
        wts = topw.reshape(-1)[order]
        start = 0
        for eid, n in enumerate(counts):
            if n:
                seg = slice(start, start + n)
                rows = tok[seg]
                acc.index_add_(0, rows, self._expert_mlp(eid, x.index_select(0, rows)).float() * wts[seg].unsqueeze(1))
            start += n
        return acc.to(x.dtype)


class GatedMLP(nn.Module):
    """One feed-forward of the gated form ``down(silu(gate(x)) * up(x))``, gate and up as one fused projection; no
    biases.  The inner width is zero-padded to a multiple of 8 (the activation kernel's 16-byte accesses)."""

    def __init__(self, hidden: int, inter: int, dtype: torch.dtype):
        super().__init__()
        self.inter, self.i_pad = inter, (inter + 7) // 8 * 8
        self.w13 = nn.Parameter(torch.zeros(2 * self.i_pad, hidden, dtype=dtype), requires_grad=False)
        self.w2 = nn.Parameter(torch.zeros(hidden, self.i_pad, dtype=dtype), requires_grad=False)
        self.w13.weight_loader = self._load_w13
        self.w2.weight_loader = self._load_w2

    def _load_w13(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        dst = param.data.narrow(0, int(shard_id) * self.i_pad, self.i_pad)
        dst.zero_()                          # (the padding included: the loader poisons fresh parameters)
        dst[:self.inter].copy_(materialize(w))

    def _load_w2(self, param: nn.Parameter, w: torch.Tensor, shard_id=None) -> None:
        param.data.zero_()
        param.data[:, :self.inter].copy_(materialize(w))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(ops.silu_and_mul(ops.linear(x, self.w13)), self.w2)


class ScoredTopKMoE(FusedMoE):
    """Routed experts of the gated form ``down(silu(gate(x)) * up(x))`` behind a router whose outputs are scored one
    by one: ``score = sigmoid(router(x))``, the ``top_k`` largest scores are chosen and ARE the weights, times
    ``route_scale``; their sum is left as it comes.  ``shared_inter > 0``: an expert of the same form that every token uses, whose
    output ``forward`` returns beside the routed sum (the caller adds both to its residual stream in one launch).

    The router is fp32 (product and scores).  On the GPU in 16-bit types the experts run as two grouped GEMMs over
    expert-sorted rows, their reduction dimensions zero-padded to the kernels' 128-deep tiles; elsewhere (fp32, CPU)
    one after the other on the library GEMM."""
    custom_routing = True

    def __init__(self, hidden: int, inter: int, num_experts: int, top_k: int, dtype: torch.dtype,
                 route_scale: float = 1.0, shared_inter: int = 0):
        super().__init__(hidden, inter, num_experts, top_k, False, dtype, expert_parallel=False, allocate_experts=False)
        if self.tp > 1:
            raise NotImplementedError("ScoredTopKMoE runs unsharded")
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top {top_k} of {num_experts} experts")
        self.quant = None
        self.route_scale = float(route_scale)
        self.gate = ReplicatedLinear(hidden, num_experts, False, dtype, quant=False)
        self.h_pad, self.i_pad = _ceil128(hidden), _ceil128(inter)
        # [gate rows ; up rows] (each padded to i_pad rows) x (reduction padded to h_pad); [hidden, i_pad]
        self.w13 = nn.Parameter(torch.zeros(num_experts, 2 * self.i_pad, self.h_pad, dtype=dtype), requires_grad=False)
        self.w2 = nn.Parameter(torch.zeros(num_experts, hidden, self.i_pad, dtype=dtype), requires_grad=False)
        self.w13.weight_loader = self._load_w13
        self.w2.weight_loader = self._load_w2
        self.shared = GatedMLP(hidden, shared_inter, dtype) if shared_inter else None

    def _load_w13(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        e, which = shard_id                  # which: 0 = gate, 1 = up
        dst = param.data[e, which * self.i_pad:(which + 1) * self.i_pad]
        dst.zero_()                          # (the padding included: the loader poisons fresh parameters)
        dst[:self.inter, :self.hidden].copy_(materialize(w))

    def _load_w2(self, param: nn.Parameter, w: torch.Tensor, shard_id) -> None:
        e, _ = shard_id
        param.data[e].zero_()
        param.data[e, :, :self.inter].copy_(materialize(w))

    def router_logits(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear_f32(x, self.gate.weight)

    def route(self, logits: torch.Tensor):
        val, topi = torch.sigmoid(logits.float()).topk(self.top_k, dim=-1)
        return val * self.route_scale, topi

    def _pad(self, x: torch.Tensor) -> torch.Tensor:
        return x if self.h_pad == self.hidden else F.pad(x, (0, self.h_pad - self.hidden))

    def _expert_mlp(self, e: int, x: torch.Tensor) -> torch.Tensor:
        return F.linear(ops.silu_and_mul(F.linear(self._pad(x), self.w13[e])), self.w2[e])

    def _grouped_tile_rows(self, x: torch.Tensor) -> int:
        if not (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and x.dim() == 2 and ops.hip_available()):
            return 0
        if self.num_experts > 512 or self.top_k > 16 or self.hidden % 16:
            return 0
        avg = x.shape[0] * self.top_k / max(1, self.num_experts)
        if avg > envs.VDAMD_MOE_GROUPED_MAX_ROWS * 2 and not torch.cuda.is_current_stream_capturing():
            return 0
        for rows in (16, 32, 64, 128):
            if avg <= rows:
                return rows
        return 128

    def decode_capturable(self, dtype: torch.dtype) -> bool:
        """Whether a decode step of this block runs without a host synchronisation (the grouped path)."""
        return (dtype in (torch.bfloat16, torch.float16) and self.hidden % 16 == 0 and self.num_experts <= 512
                and self.top_k <= 16)

    def forward(self, x: torch.Tensor, reduce: bool = True, staged: bool = False, deferred: bool = False):
        """Returns ``(routed sum, shared expert's output or None)``."""
        logits = self.router_logits(x)
        shared = self.shared(x) if self.shared is not None else None
        tile_rows = self._grouped_tile_rows(x)
        if tile_rows:
            topw, topi = ops.moe_topk_grouped(logits, None, self.top_k, 1, 1, True, False, False, self.route_scale)
            src_row, inv, tiles = ops.moe_align_fused(topi, self.num_experts, tile_rows, 0, -1)
            xs = self._pad(x).index_select(0, src_row)
            h = ops.grouped_linear(xs, tiles, tile_rows, weight=self.w13)
            y = ops.grouped_linear(ops.silu_and_mul(h), tiles, tile_rows, weight=self.w2)
            return ops.moe_combine(y, topw, topi, inv, 0, -1), shared
        topw, topi = self.route(logits)
        acc = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        flat_e = topi.reshape(-1)
        order = flat_e.argsort(stable=True)
        counts = torch.bincount(flat_e, minlength=self.num_experts).tolist()
        tok = order // self.top_k
        wts = topw.reshape(-1)[order]
        start = 0
        for eid, n in enumerate(counts):
            if n:
                seg = slice(start, start + n)
                rows = tok[seg]
                acc.index_add_(0, rows, self._expert_mlp(eid, x.index_select(0, rows)).float() * wts[seg].unsqueeze(1))
            start += n
        return acc.to(x.dtype), shared
