"""Nalasun: a decoder-only model with learned positions whose layers put one of three sequence mixers and a sparse
feed-forward around an fp32 residual stream, every mixer reading its normed input through a short causal convolution.

``x = embed[token] + pos[position]``; per layer ``h = norm1(x)``, ``h <- h + conv(h)`` (a per-channel causal
convolution over time, ``canon.taps`` taps, no bias, no activation), ``x <- x + mixer(h)``, then where the layer has a
feed-forward ``x <- x + ff(norm2(x))``; RMS norms with plain gains.  ``config.json`` lists the layers one by one
(``layers[i] = {type, mixer{...}, mlp{...} | null}``), so order, heads, sizes and constants differ from layer to layer
and from model to model.  A final norm and the embedding table itself give fp32 logits.

Mixers
  * ``attention`` - ``layers.attention.CrossedBiasAttention``: grouped-query softmax attention without rotation;
    q and k have biases and are RMS-normed over ALL their heads at once; the un-normed key projection doubles as the value (no
    value projection); q is scaled by ``1 + coef * ln(floor((p + 1) / every) + 1)`` at position ``p``; the score is
    ``q.k * scale - r1[h] * ln(1 + r2[h] * (i - j))``; after the softmax the heads' weights are mixed by a learned
    ``[H, H]`` matrix.
  * ``channel_delta`` - ``layers.linear_attention.GatedDeltaRule`` behind convolved, SiLU'd projections (unit-length
    q and k, a decay per head and key channel from a low-rank projection, per-head RMS norm times a low-rank sigmoid
    gate).
  * ``mamba2`` - ``layers.linear_attention.SelectiveStateSpace``: one projection gives ``[z | x | B | C | dt]``;
    x, B and C pass a convolution with bias and SiLU; the recurrence's output is multiplied by ``silu(z)`` and THEN
    RMS-normed in ``norm_groups`` equal parts.

Feed-forward: ``layers.moe.ScoredTopKMoE`` (gated SiLU experts, sigmoid scores as weights times ``router.scale``, an
always-on shared expert).

Tensor and pipeline parallelism are not implemented for this family (the norms reduce over whole rows and the
recurrent state is not sharded).
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..parallel.state import get_pp_group, get_tensor_model_parallel_world_size
from .layers.attention import Attention, CrossedBiasAttention, ResidualRMSNorm, get_forward_context
from .layers.linear import ColumnParallelLinear, RowParallelLinear, VocabParallelEmbedding
from .layers.linear_attention import DeltaRuleMixer, SelectiveStateSpace
from .layers.moe import ScoredTopKMoE
from .layers.short_conv import ShortConv, SlotState
from .utils import IntermediateTensors, materialize


def _f32(*shape: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(shape, dtype=torch.float32), requires_grad=False)


def _taps(shapes: Dict[str, Tuple[int, ...]], tensor: str, stated) -> int:
    """Taps of a convolution: the checkpoint tensor's second dimension where there is one, else what the config
    states."""
    shape = shapes.get(tensor)
    return int(shape[1]) if shape is not None and len(shape) == 2 else int(stated or 0)


def _conv_rows(md, positions):
    """The sequence of every row of the step (None in a pure decode batch: row ``t`` is sequence ``t``)."""
    return None if md.num_prefills == 0 else md.token_rows(positions)[0]


# ---------------------------------------------------------------------------------------------------- mixers
class SharedValueAttentionMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype):
        super().__init__()
        self.heads, self.kv_heads, self.dim = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"])
        if self.heads % self.kv_heads:
            raise ValueError(f"layer {layer_idx}: {self.heads} query heads do not divide over {self.kv_heads} kv heads")
        if int(m.get("vdim") or self.dim) != self.dim:
            raise ValueError(f"layer {layer_idx}: the values are the keys, so vdim must equal dim ({self.dim})")
        self.eps = eps
        qt = m.get("q_temp") or {}
        self.temp_coef, self.temp_every = float(qt.get("coef") or 0.0), int(qt.get("every") or 0)
        if self.temp_coef == 0.0:
            self.temp_every = 0
        qs, ks = self.heads * self.dim, self.kv_heads * self.dim
        self.proj = ColumnParallelLinear(width, [qs, ks], True, dtype)
        self.q_norm, self.k_norm = _f32(qs), _f32(ks)
        self.attn = CrossedBiasAttention(self.heads, self.dim, self.kv_heads, float(m.get("scale") or self.dim ** -0.5),
                                         layer_idx)
        self.o = RowParallelLinear(qs, width, False, dtype)

    def state_layers(self) -> List[SlotState]:
        return []

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_forward_context()
        md = ctx.attn_metadata
        x = self.proj(h)
        attn = self.attn
        q = ops.joint_norm_cache(x, self.heads, self.kv_heads, self.dim, self.q_norm, self.k_norm, self.eps,
                                 ctx.positions, self.temp_coef, self.temp_every,
                                 None if md is None else attn.k_cache, None if md is None else attn.v_cache,
                                 None if md is None else md.slot_mapping)
        return self.o(attn.forward_cached(q))


class ChannelDeltaMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype,
                 shapes: Dict[str, Tuple[int, ...]]):
        super().__init__()
        m = dict(m)
        # the widths of the two low-rank projections are sizes only the tensors state
        for key, tensor in (("decay_rank", "a1"), ("gate_rank", "g1")):
            if m.get(key) is None:
                shape = shapes.get(f"l{layer_idx}.mix.{tensor}")
                if shape is None:
                    raise ValueError(f"layer {layer_idx}: neither the config ({key}) nor a checkpoint tensor "
                                     f"(mix.{tensor}) gives the width of the low-rank projection")
                m[key] = int(shape[0])
        m["conv"] = _taps(shapes, f"l{layer_idx}.mix.q.conv", m.get("conv")) or 1
        self.dtype = dtype
        self.inner = DeltaRuleMixer(width, m, eps, layer_idx, dtype, 1, 1.0)
        self.o = RowParallelLinear(self.inner.out_cols, width, False, dtype)

    def state_layers(self) -> List[SlotState]:
        return [self.inner.conv_states[0], self.inner.rule_states[0]]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        heads = torch.empty((h.shape[0], self.inner.out_cols), dtype=self.dtype, device=h.device)
        self.inner(h, 0, heads)
        return self.o(heads)


class StateSpaceMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype,
                 shapes: Dict[str, Tuple[int, ...]]):
        super().__init__()
        heads, vdim, n, groups = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups") or 1)
        self.inner_cols, self.eps, self.dtype = heads * vdim, eps, dtype
        parts = int(m.get("norm_groups") or 1)
        if parts < 1 or self.inner_cols % parts:
            raise ValueError(f"layer {layer_idx}: {self.inner_cols} channels do not split into {parts} equal norm groups")
        self.norm_group = self.inner_cols // parts
        self.ssm = SelectiveStateSpace(heads, groups, vdim, n, layer_idx)
        bc = groups * n
        # [z | x | B | C | dt]
        self.proj = ColumnParallelLinear(width, [self.inner_cols, self.inner_cols, bc, bc, heads], False, dtype)
        self.conv = ShortConv([self.inner_cols, bc, bc], _taps(shapes, f"l{layer_idx}.mix.conv", m.get("conv")) or 1,
                              dtype, bias=True)
        self.conv_state = SlotState((max(self.conv.taps - 1, 1), self.conv.channels))
        self.ssm_state = SlotState(self.ssm.per_slot_shape(), torch.float32)
        self.norm = _f32(self.inner_cols)
        self.o = RowParallelLinear(self.inner_cols, width, False, dtype)

    def state_layers(self) -> List[SlotState]:
        return [self.conv_state, self.ssm_state]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_forward_context()
        md = ctx.attn_metadata
        u = self.proj(h)
        if md is None:                    # memory-profiling pass: no state
            return self.o(u[:, :self.inner_cols].contiguous())
        c = self.conv.channels
        lo = self.inner_cols
        xbc = ops.short_conv_act(u[:, lo:], c, self.conv.weight_t, self.conv_state.state, md.state_slots,
                                 md.query_start_loc, md.seq_lens, _conv_rows(md, ctx.positions), ctx.positions, True,
                                 md.num_prefills > 0, self.conv.bias)
        y = self.ssm(xbc, u[:, lo + c:], self.ssm_state.state)
        return self.o(ops.act_gate_group_norm(y, u[:, :lo], self.norm, self.eps, self.norm_group, self.dtype))


def _make_mixer(width: int, spec: dict, eps: float, layer_idx: int, dtype: torch.dtype,
                shapes: Dict[str, Tuple[int, ...]]) -> nn.Module:
    kind, m = spec.get("type"), spec["mixer"]
    if kind == "attention":
        return SharedValueAttentionMixer(width, m, eps, layer_idx, dtype)
    if kind == "channel_delta":
        return ChannelDeltaMixer(width, m, eps, layer_idx, dtype, shapes)
    if kind == "mamba2":
        return StateSpaceMixer(width, m, eps, layer_idx, dtype, shapes)
    raise ValueError(f"layer {layer_idx}: unknown mixer type {kind!r}")


def _make_mlp(width: int, mlp: dict, layer_idx: int, dtype: torch.dtype) -> nn.Module:
    kind = mlp.get("kind", "moe")
    if kind != "moe":
        raise ValueError(f"layer {layer_idx}: unknown feed-forward kind {kind!r}")
    r, s = mlp["router"], mlp.get("shared")
    return ScoredTopKMoE(width, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), dtype,
                         route_scale=float(r.get("scale", 1.0)), shared_inter=int(s["ff"]) if s else 0)


class NalasunLayer(nn.Module):
    def __init__(self, width: int, spec: dict, eps: float, taps: int, layer_idx: int, dtype: torch.dtype,
                 shapes: Dict[str, Tuple[int, ...]]):
        super().__init__()
        self.width = width
        self.norm1 = ResidualRMSNorm(width, eps, dtype)
        # the convolution in front of the mixer: its last taps - 1 inputs are per-request state in every layer
        self.canon = ShortConv([width], taps, dtype) if taps > 0 else None
        self.canon_state = SlotState((max(taps - 1, 1), width)) if taps > 0 else None
        self.mix = _make_mixer(width, spec, eps, layer_idx, dtype, shapes)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            self.norm2 = ResidualRMSNorm(width, eps, dtype)
            self.mlp = _make_mlp(width, mlp, layer_idx, dtype)

    def state_layers(self) -> List[SlotState]:
        return ([self.canon_state] if self.canon_state is not None else []) + self.mix.state_layers()

    def forward(self, x: torch.Tensor, h: torch.Tensor, then: ResidualRMSNorm) -> torch.Tensor:
        """``x``: fp32 residual stream (updated in place), ``h = norm1(x)``; returns ``then(x)`` after this layer.
        Every residual add and the norm that follows it are one launch."""
        ctx = get_forward_context()
        md = ctx.attn_metadata
        if self.canon is not None and md is not None:
            h = ops.short_conv_act(h, self.width, self.canon.weight_t, self.canon_state.state, md.state_slots,
                                   md.query_start_loc, md.seq_lens, _conv_rows(md, ctx.positions), ctx.positions,
                                   False, md.num_prefills > 0, None, True)
        y = self.mix(h)
        if self.mlp is None:
            return then.add(x, y)
        routed, shared = self.mlp(self.norm2.add(x, y))
        return then.add(x, routed, shared)


class NalasunForCausalLM(nn.Module):
    has_request_state = True          # convolutions and recurrent layers remember a state per request: no prefix reuse
    residual_dtype = torch.float32

    def __init__(self, vllm_config: VllmConfig):
        super().__init__()
        mc = vllm_config.model_config
        cfg, dtype = mc.hf_config, mc.torch_dtype
        self.cfg, self.dtype = cfg, dtype
        if get_tensor_model_parallel_world_size() > 1 or get_pp_group().world_size > 1:
            raise NotImplementedError("Nalasun runs on one device: its norms reduce over whole rows and its recurrent "
                                      "state is not sharded")
        self.is_first = self.is_last = True
        width, eps = int(cfg["width"]), float((cfg.get("norm") or {}).get("eps", 1e-5))
        specs = cfg["layers"]
        if not specs:
            raise ValueError("a Nalasun model needs at least one layer")
        self.width, self.eps, self.vocab = width, eps, int(cfg["vocab"])
        self.start_layer, self.end_layer = 0, len(specs)
        self.embed = VocabParallelEmbedding(self.vocab, width, dtype)
        from ..config import resolve_model_path
        from .loader import checkpoint_tensor_shapes
        shapes = {} if mc.load_format == "dummy" else checkpoint_tensor_shapes(resolve_model_path(mc.model))
        taps = _taps(shapes, "l0.canon1", (cfg.get("canon") or {}).get("taps"))
        positions = int(cfg.get("max_positions") or (shapes.get("pos") or (0,))[0])
        if positions <= 0:
            raise ValueError("neither the config (max_positions) nor a checkpoint tensor (pos) gives the number of positions")
        self.pos = nn.Embedding(positions, width, dtype=dtype)
        self.pos.weight.requires_grad_(False)
        self.layers = nn.ModuleList(NalasunLayer(width, s, eps, taps, i, dtype, shapes) for i, s in enumerate(specs))
        self.final_norm = ResidualRMSNorm(width, eps, dtype)
        self.trace_residual: Optional[List[torch.Tensor]] = None      # tests: the residual stream after every layer

    def rebind_buffers(self) -> None:
        return None

    def attention_layers(self) -> List[Attention]:
        return [l.mix.attn for l in self.layers if isinstance(l.mix, SharedValueAttentionMixer)]

    def state_layers(self) -> List[SlotState]:
        out: List[SlotState] = []
        for l in self.layers:
            out += l.state_layers()
        return out

    def decode_capturable(self) -> bool:
        return all(l.mlp.decode_capturable(self.dtype) for l in self.layers if l.mlp is not None)

    def forward(self, input_ids, positions, intermediate: Optional[IntermediateTensors] = None):
        x = ops.embed_positions(input_ids, positions, self.embed.weight, self.pos.weight)
        n = len(self.layers)
        h = self.layers[0].norm1(x)
        for i, layer in enumerate(self.layers):
            h = layer(x, h, self.layers[i + 1].norm1 if i + 1 < n else self.final_norm)
            if self.trace_residual is not None:
                self.trace_residual.append(x.clone())
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear_f32(hidden, self.embed.weight)[..., :self.vocab]

    # ------------------------------------------------------------ weights
    _ATTENTION = {"q": ("proj.weight", 0), "k": ("proj.weight", 1), "q.b": ("proj.bias", 0), "k.b": ("proj.bias", 1),
                  "q.norm": ("q_norm", None), "k.norm": ("k_norm", None), "r1": ("attn.bias_scale", None),
                  "r2": ("attn.bias_rate", None), "talk": ("attn.talk", None), "o": ("o.weight", None)}
    _DELTA = {"q": ("inner.proj.weight", 0), "k": ("inner.proj.weight", 1), "v": ("inner.proj.weight", 2),
              "b": ("inner.proj.weight", 3), "a1": ("inner.proj.weight", 4), "g1": ("inner.proj.weight", 5),
              "a2": ("inner.a2.weight", None), "g2": ("inner.g2.weight", None),
              "q.conv": ("inner.conv.weight", 0), "k.conv": ("inner.conv.weight", 1), "v.conv": ("inner.conv.weight", 2),
              "A_log": ("inner.rule.a_log", None), "dt_bias": ("inner.rule.dt_bias", None),
              "norm": ("inner.norm", None), "o": ("o.weight", None)}
    _SSM = {"in": ("proj.weight", None), "conv": ("conv.weight", None), "conv.b": ("conv.bias", None),
            "dt_bias": ("ssm.dt_bias", None), "A_log": ("ssm.a_log", None), "D": ("ssm.d_skip", None),
            "norm": ("norm", None), "o": ("o.weight", None)}

    def _target(self, name: str):
        """Checkpoint tensor name -> (parameter name, shard of a fused parameter)."""
        top = {"embed": "embed.weight", "pos": "pos.weight", "final.norm": "final_norm.weight"}
        if name in top:
            return top[name], None
        if not name.startswith("l"):
            return None
        idx, _, rest = name[1:].partition(".")
        if not idx.isdigit() or int(idx) >= len(self.layers):
            return None
        layer, base = self.layers[int(idx)], f"layers.{idx}."
        flat = {"norm1": "norm1.weight", "norm2": "norm2.weight", "canon1": "canon.weight"}
        if rest in flat:
            return base + flat[rest], None
        kind, _, leaf = rest.partition(".")
        if kind == "mix":
            table = (self._ATTENTION if isinstance(layer.mix, SharedValueAttentionMixer)
                     else self._DELTA if isinstance(layer.mix, ChannelDeltaMixer) else self._SSM)
            if leaf not in table:
                return None
            p, shard = table[leaf]
            return base + "mix." + p, shard
        if kind != "mlp" or layer.mlp is None:
            return None
        if leaf == "router":
            return base + "mlp.gate.weight", None
        e, _, part = leaf.partition(".")
        which = {"gate": 0, "up": 1}
        if e == "shared" and layer.mlp.shared is not None:
            if part in which:
                return base + "mlp.shared.w13", which[part]
            return (base + "mlp.shared.w2", None) if part == "down" else None
        if e[:1] == "e" and e[1:].isdigit() and int(e[1:]) < layer.mlp.num_experts:
            if part in which:
                return base + "mlp.w13", (int(e[1:]), which[part])
            if part == "down":
                return base + "mlp.w2", (int(e[1:]), 0)
        return None

    def map_weight_name(self, name: str) -> Optional[str]:
        t = self._target(name)
        return None if t is None else t[0]

    def _owns_layer(self, name: str) -> bool:
        return True

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        params: Dict[str, nn.Parameter] = dict(self.named_parameters())
        loaded = []
        for name, w in weights:
            t = self._target(name)
            if t is None or t[0] not in params:
                continue
            p, shard = params[t[0]], t[1]
            loader = getattr(p, "weight_loader", None)
            if loader is not None:
                loader(p, w, shard)
            else:
                w = materialize(w)
                assert w.numel() == p.numel(), (name, tuple(w.shape), tuple(p.shape))
                p.data.copy_(w.reshape(p.shape))
            loaded.append(name)
        return loaded


def weight_shapes(c: dict) -> Dict[str, Tuple[int, ...]]:
    """Checkpoint tensor names and shapes of a Nalasun config (for the random-weight loader); a ``channel_delta``
    mixer has to state ``decay_rank`` and ``gate_rank`` then."""
    width, vocab = int(c["width"]), int(c["vocab"])
    taps = int((c.get("canon") or {}).get("taps") or 0)
    out: Dict[str, Tuple[int, ...]] = {"embed": (vocab, width), "pos": (int(c["max_positions"]), width)}
    for i, spec in enumerate(c["layers"]):
        m, p, q = spec["mixer"], f"l{i}.", f"l{i}.mix."
        out[p + "norm1"] = (width,)
        if taps:
            out[p + "canon1"] = (width, taps)
        kind = spec["type"]
        if kind == "attention":
            heads, kvh, dim = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"])
            out[q + "q"], out[q + "q.b"], out[q + "q.norm"] = (heads * dim, width), (heads * dim,), (heads * dim,)
            out[q + "k"], out[q + "k.b"], out[q + "k.norm"] = (kvh * dim, width), (kvh * dim,), (kvh * dim,)
            out[q + "r1"], out[q + "r2"], out[q + "talk"] = (heads,), (heads,), (heads, heads)
            out[q + "o"] = (width, heads * dim)
        elif kind == "channel_delta":
            heads, kvh = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
            dim, vdim, taps_m = int(m["dim"]), int(m.get("vdim") or m["dim"]), int(m.get("conv") or 1)
            for nm, rows in (("q", kvh * dim), ("k", kvh * dim), ("v", heads * vdim)):
                out[q + nm], out[q + nm + ".conv"] = (rows, width), (rows, taps_m)
            dr, gr = int(m["decay_rank"]), int(m["gate_rank"])
            out[q + "b"], out[q + "A_log"], out[q + "norm"] = (heads, width), (heads,), (vdim,)
            out[q + "a1"], out[q + "a2"], out[q + "dt_bias"] = (dr, width), (heads * dim, dr), (heads * dim,)
            out[q + "g1"], out[q + "g2"], out[q + "o"] = (gr, width), (heads * vdim, gr), (width, heads * vdim)
        elif kind == "mamba2":
            heads, vdim, n, g = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups") or 1)
            inner, ch = heads * vdim, heads * vdim + 2 * g * n
            out[q + "in"] = (2 * inner + 2 * g * n + heads, width)
            out[q + "conv"], out[q + "conv.b"] = (ch, int(m.get("conv") or 1)), (ch,)
            out[q + "dt_bias"], out[q + "A_log"], out[q + "D"] = (heads,), (heads,), (heads,)
            out[q + "norm"], out[q + "o"] = (inner,), (width, inner)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = spec.get("mlp")
        if mlp:
            out[p + "norm2"] = (width,)
            ff = int(mlp["expert"]["ff"])
            names = [f"e{e}" for e in range(int(mlp["router"]["experts"]))]
            sizes = [ff] * len(names)
            if mlp.get("shared"):
                names.append("shared")
                sizes.append(int(mlp["shared"]["ff"]))
            for nm, f in zip(names, sizes):
                out[f"{p}mlp.{nm}.gate"], out[f"{p}mlp.{nm}.up"], out[f"{p}mlp.{nm}.down"] = (f, width), (f, width), (width, f)
            out[p + "mlp.router"] = (int(mlp["router"]["experts"]), width)
    out["final.norm"] = (width,)
    return out


def random_weight(name: str, shape: Tuple[int, ...], gen: torch.Generator, device, dtype) -> torch.Tensor:
    """A plausible random value for a checkpoint tensor (projections that keep the variance, norm gains around one,
    small biases, decays spread over (0, 1), a head-mixing matrix near the identity)."""
    def uni(lo: float, hi: float) -> torch.Tensor:
        return lo + (hi - lo) * torch.rand(shape, generator=gen, device=device, dtype=torch.float32)
    leaf = name.rsplit(".", 1)[-1]
    if leaf in ("norm1", "norm2", "norm", "D") or name == "final.norm":
        w = uni(0.8, 1.2)
    elif leaf == "talk":
        w = torch.eye(shape[0], device=device, dtype=torch.float32) + uni(-0.2, 0.2)
    elif leaf in ("r1", "r2"):
        w = uni(0.05, 1.0)
    elif leaf == "dt_bias":
        w = uni(-3.0, -1.0)
    elif leaf == "b" and len(shape) == 1:
        w = uni(-0.5, 0.5)
    elif leaf == "A_log":
        w = uni(-2.0, 0.5)
    elif leaf in ("conv", "canon1"):
        w = uni(-0.6, 0.6)
    elif name in ("embed", "pos"):
        w = uni(-1.0, 1.0)
    else:
        s = (3.0 / shape[-1]) ** 0.5
        w = uni(-s, s)
    return w.to(dtype)
