"""Gosizen: a decoder-only model whose layers add a sequence mixer and a feed-forward, both reading ONE normed input,
to an fp32 residual stream, with a per-layer input looked up by token and a block of layers that runs several times.

``x = embed[token]``; per layer ``h = norm1(x)``, ``x <- x + mixer(h) + ff(h)`` (RMS norms whose stored weight is the
gain minus one); then, when the model has a token side input, ``e = side_embed[token][layer's part]``,
``y = proj(gelu_tanh(gate(x)) * e)``, ``x <- x + rms_norm(y) * side_norm``.  ``config.json`` lists the layers one by one
(``layers[i] = {type, mixer{...}, mlp{...} | null}``), so order, heads, sizes, windows and constants differ from layer
to layer and from model to model.  ``loop = {start, stop, times}``: layers ``start .. stop - 1`` run ``times`` times
over the same weights; before each pass ``x <- W_in [x ; embed[token]] + step[pass]``; every pass keeps its own cache
rows and state.  A final norm, the head and a tanh cap give fp32 logits.

Mixers
  * ``latent_attention`` - ``layers.attention.RowLatentAttention``: keys and values are expansions of one cached row
    per token ``[RMS-normed latent (kv_rank) | rotated key part shared by the heads (rot_dim)]``, the expansions
    folded into the query and the output; the query itself comes through a normed latent (``q_rank``); rotation over
    neighbouring pairs; a sliding window; a sink in the softmax denominator; a sigmoid gate per head.
  * ``parallel`` - two mixers side by side on the same input, ``left_scale * left + right_scale * right``, their
    output projections fused into one GEMM over ``[left heads | right heads]``:
    left = ``layers.attention.WindowBiasAttention`` with a chunked mask behind ``layers.short_conv.ShortConv``
    (projections with biases, convolution, rotation over pairs half the rotated width apart with wavelength-banded
    frequency scaling, a sink, an element-wise sigmoid gate);
    right = ``layers.linear_attention.GatedDeltaRule`` (convolution + SiLU on q / k / v, unit-length q and k, a decay
    per head and key channel from a low-rank projection, per-head RMS norm times a low-rank sigmoid gate).

Feed-forwards: ``dense`` - ``down(gelu_tanh(up(h)))``; ``moe`` - ``layers.moe.BiasedTopKMoE`` (plain experts with the
exact GELU, a router with a bias, softmax over the chosen).

Tensor and pipeline parallelism are not implemented for this family (the norms reduce over whole rows and the
recurrent state is not sharded).
"""
from __future__ import annotations

from typing import Dict, Iterable, List, NamedTuple, Optional, Tuple

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..parallel.state import get_pp_group, get_tensor_model_parallel_world_size
from .layers.attention import (Attention, ResidualRMSNorm, RowLatentAttention, WindowBiasAttention, get_forward_context,
                               rotary_frequencies)
from .layers.linear import ColumnParallelLinear, ReplicatedLinear, RowParallelLinear, VocabParallelEmbedding
from .layers.linear_attention import DeltaRuleMixer
from .layers.moe import BiasedTopKMoE
from .layers.short_conv import ShortConv, SlotState
from .utils import IntermediateTensors, materialize


def _f32(*shape: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(shape, dtype=torch.float32), requires_grad=False)


def _mask_size(m: dict) -> int:
    return int((m.get("mask") or {}).get("size") or 0)


class Run(NamedTuple):
    """One execution of a layer in a forward pass."""
    layer: int
    index: int          # which of the layer's caches and states it uses (its pass number; 0 outside the loop)
    opens: int          # the pass this run opens (the loop's input mix comes first), or -1


def layer_runs(num_layers: int, loop: Optional[dict]) -> List[Run]:
    if not loop:
        return [Run(i, 0, -1) for i in range(num_layers)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if not (0 <= start < stop <= num_layers) or times < 1:
        raise ValueError(f"loop {loop} does not fit {num_layers} layers")
    runs = [Run(i, 0, -1) for i in range(start)]
    for t in range(times):
        runs += [Run(i, t, t if i == start else -1) for i in range(start, stop)]
    return runs + [Run(i, 0, -1) for i in range(stop, num_layers)]


# ---------------------------------------------------------------------------------------------------- mixers
class GatedLatentMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype, passes: int):
        super().__init__()
        self.heads, self.nope, self.rope = int(m["heads"]), int(m["dim"]), int(m["rot_dim"])
        self.vdim, self.rank, self.q_rank = int(m.get("vdim") or m["dim"]), int(m["kv_rank"]), int(m["q_rank"])
        self.eps, self.dtype = eps, dtype
        rot = m.get("rot") or {}
        dims = int(rot.get("dims") or self.rope)
        if dims > self.rope or dims % 2:
            raise ValueError(f"layer {layer_idx}: {dims} rotated dimensions in a part of {self.rope}")
        freq, _ = rotary_frequencies(dims, float(rot.get("base", 10000.0)), rot.get("scaling"))
        self.register_buffer("inv_freq", freq, persistent=False)
        self.proj = ColumnParallelLinear(width, [self.q_rank, self.rank + self.rope, self.heads], False, dtype)
        self.dq_norm, self.dkv_norm = _f32(self.q_rank), _f32(self.rank)
        self.uq = ColumnParallelLinear(self.q_rank, [self.heads * (self.nope + self.rope)], False, dtype)
        self.uk = nn.Parameter(torch.empty(self.heads * self.nope, self.rank, dtype=dtype), requires_grad=False)
        self.uv = nn.Parameter(torch.empty(self.heads * self.vdim, self.rank, dtype=dtype), requires_grad=False)
        self.sink = _f32(self.heads)
        scale = float(m.get("scale") or (self.nope + self.rope) ** -0.5)
        self.attn = nn.ModuleList(RowLatentAttention(self.heads, self.rank, self.rope, scale, layer_idx, dtype=dtype,
                                                     window=_mask_size(m), sink=self.sink, interleaved=True)
                                  for _ in range(passes))
        self.o = RowParallelLinear(self.heads * self.vdim, width, False, dtype)
        self._folded = None

    def _folded_weights(self):
        """``uk`` as ``[H, nope, rank]`` (multiplied into the query) and ``uv`` as ``[H, rank, vdim]`` (applied to
        the attention output)."""
        if self._folded is None:
            self._folded = (self.uk.data.view(self.heads, self.nope, self.rank),
                            self.uv.data.view(self.heads, self.vdim, self.rank).transpose(1, 2).contiguous())
        return self._folded

    def forward(self, h: torch.Tensor, index: int) -> torch.Tensor:
        t = h.shape[0]
        x = self.proj(h)
        cq = ops.rms_norm_to(x[:, :self.q_rank], self.dq_norm, self.eps, self.dtype)
        q = self.uq(cq).view(t, self.heads, self.nope + self.rope)
        latent = x[:, self.q_rank:self.q_rank + self.rank + self.rope]
        gate = x[:, self.q_rank + self.rank + self.rope:]
        w_uk, w_uv_t = self._folded_weights()
        q_lat = torch.bmm(q[..., :self.nope].transpose(0, 1), w_uk)                    # [H, T, rank]
        o_lat = self.attn[index].forward_latent(q, self.nope, q_lat, latent, self.dkv_norm, self.eps, self.inv_freq,
                                                1.0, gate)
        o = torch.bmm(o_lat.transpose(0, 1), w_uv_t).transpose(0, 1).reshape(t, self.heads * self.vdim)
        return self.o(o)


class ChunkedConvAttention(nn.Module):
    """The left half of a parallel mixer; writes ``scale * gated heads`` into the columns it is given."""

    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype, passes: int, scale: float):
        super().__init__()
        self.heads, self.kv_heads = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
        self.dim, self.vdim = int(m["dim"]), int(m.get("vdim") or m["dim"])
        if self.heads % self.kv_heads:
            raise ValueError(f"layer {layer_idx}: {self.heads} query heads do not divide over {self.kv_heads} kv heads")
        self.eps, self.out_scale = eps, float(scale)
        qs, ks, vs = self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim
        self.channels, self.out_cols = qs + ks + vs, self.heads * self.vdim
        self.proj = ColumnParallelLinear(width, [qs, ks, vs, self.out_cols], True, dtype)
        self.conv = ShortConv([qs, ks, vs], int(m.get("conv") or 1), dtype)
        self.conv_states = [SlotState((max(self.conv.taps - 1, 1), self.channels)) for _ in range(passes)]
        rot = m.get("rot") or {}
        dims = int(rot.get("dims") or 0)
        if dims > self.dim or dims % 2:
            raise ValueError(f"layer {layer_idx}: {dims} rotated dimensions in heads of {self.dim}")
        freq, _ = rotary_frequencies(dims, float(rot.get("base", 10000.0)), rot.get("scaling")) if dims else (None, 1.0)
        self.register_buffer("inv_freq", freq, persistent=False)
        self.sink = _f32(self.heads)
        self.attn = nn.ModuleList(WindowBiasAttention(self.heads, self.dim, self.vdim, self.kv_heads,
                                                      float(m.get("scale") or self.dim ** -0.5), layer_idx,
                                                      distance_bias=False, sink=self.sink, chunk=_mask_size(m))
                                  for _ in range(passes))

    def finalize_weights(self) -> None:
        self.proj.bias.data[self.channels:] = 0          # the gate projection has no bias

    def forward(self, h: torch.Tensor, index: int, out: torch.Tensor) -> None:
        ctx = get_forward_context()
        md = ctx.attn_metadata
        x = self.proj(h)
        if md is None:                    # memory-profiling pass: no cache, no state
            out.zero_()
            return
        attn = self.attn[index]
        rows = None if md.num_prefills == 0 else md.token_rows(ctx.positions)[0]
        q, _ = ops.conv_norm_cache(
            x, self.conv.weight_t, self.conv_states[index].state, md.state_slots, md.query_start_loc, md.seq_lens, rows,
            ctx.positions, self.heads, self.kv_heads, self.dim, self.vdim, None, None, self.eps, None, None, False,
            attn.k_cache, attn.v_cache, md.slot_mapping, md.num_prefills > 0, self.inv_freq)
        ops.sigmoid_mul(attn.forward_cached(q), x[:, self.channels:], self.out_scale, out=out)


class ParallelMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype, passes: int,
                 shapes: Dict[str, Tuple[int, ...]]):
        super().__init__()
        right = dict(m["right"])
        # the widths of the two low-rank projections are sizes only the tensors state
        for key, tensor in (("decay_rank", "a1"), ("gate_rank", "g1")):
            if right.get(key) is None:
                shape = shapes.get(f"l{layer_idx}.mix.right.{tensor}")
                if shape is None:
                    raise ValueError(f"layer {layer_idx}: neither the config ({key}) nor a checkpoint tensor "
                                     f"(mix.right.{tensor}) gives the width of the low-rank projection")
                right[key] = int(shape[0])
        self.left = ChunkedConvAttention(width, m["left"], eps, layer_idx, dtype, passes, float(m.get("left_scale", 1.0)))
        self.right = DeltaRuleMixer(width, right, eps, layer_idx, dtype, passes, float(m.get("right_scale", 1.0)))
        self.dtype = dtype
        self.o = RowParallelLinear(self.left.out_cols + self.right.out_cols, width, False, dtype)

    def forward(self, h: torch.Tensor, index: int) -> torch.Tensor:
        nl = self.left.out_cols
        heads = torch.empty((h.shape[0], nl + self.right.out_cols), dtype=self.dtype, device=h.device)
        self.left(h, index, heads[:, :nl])
        self.right(h, index, heads[:, nl:])
        return self.o(heads)


# ---------------------------------------------------------------------------------------------------- feed-forwards
class GeluMLP(nn.Module):
    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        self.up = ColumnParallelLinear(width, [ff], False, dtype)
        self.down = RowParallelLinear(ff, width, False, dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.gelu(self.up(h), True))


def _make_mlp(width: int, mlp: dict, layer_idx: int, dtype: torch.dtype) -> nn.Module:
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return GeluMLP(width, int(mlp["ff"]), dtype)
    if kind != "moe":
        raise ValueError(f"layer {layer_idx}: unknown feed-forward kind {kind!r}")
    r = mlp["router"]
    return BiasedTopKMoE(width, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), dtype, activation="gelu")


class TokenSide(nn.Module):
    """A layer's input by token: ``proj(gelu_tanh(gate(x)) * table[token][col : col + dim])``, RMS-normed with a
    plain weight before it joins the residual stream (the caller fuses that with the next layer's norm)."""

    def __init__(self, width: int, dim: int, col: int, dtype: torch.dtype):
        super().__init__()
        self.col = col
        self.gate = ReplicatedLinear(width, dim, False, dtype)
        self.proj = ReplicatedLinear(dim, width, False, dtype)
        self.norm = _f32(width)

    def forward(self, xb: torch.Tensor, table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        return self.proj(ops.gelu_mul_rows(self.gate(xb), table, ids, self.col))


class GosizenLayer(nn.Module):
    def __init__(self, width: int, spec: dict, eps: float, layer_idx: int, dtype: torch.dtype, passes: int,
                 side_dim: int, shapes: Dict[str, Tuple[int, ...]]):
        super().__init__()
        self.eps, self.dtype = eps, dtype
        self.norm1 = ResidualRMSNorm(width, eps, dtype, offset=1.0)
        kind, m = spec.get("type"), spec["mixer"]
        if kind == "latent_attention":
            self.mix = GatedLatentMixer(width, m, eps, layer_idx, dtype, passes)
        elif kind == "parallel":
            self.mix = ParallelMixer(width, m, eps, layer_idx, dtype, passes, shapes)
        else:
            raise ValueError(f"layer {layer_idx}: unknown mixer type {kind!r}")
        mlp = spec.get("mlp")
        self.mlp = _make_mlp(width, mlp, layer_idx, dtype) if mlp is not None else None
        self.side = TokenSide(width, side_dim, layer_idx * side_dim, dtype) if side_dim else None

    def forward(self, x: torch.Tensor, h: torch.Tensor, index: int, ids: torch.Tensor, table: Optional[torch.Tensor],
                then: Optional[ResidualRMSNorm]) -> torch.Tensor:
        """``x``: fp32 residual stream (updated in place), ``h = norm1(x)``.  Returns ``then(x)`` after this layer,
        or with ``then`` None the stream itself in the model dtype.  The residual adds and the norm that follows are
        one launch each."""
        y = self.mix(h, index)
        f = self.mlp(h) if self.mlp is not None else None
        if self.side is None:
            if then is None:
                return ops.add_rms_norm_to(x, y, f, None, self.eps, self.dtype, normed=False)
            return then.add(x, y, f)
        s = self.side(ops.add_rms_norm_to(x, y, f, None, self.eps, self.dtype, normed=False), table, ids)
        if then is None:
            return ops.norm_add_norm(s, self.side.norm, x, None, self.eps, self.dtype, next_normed=False)
        return then.after(s, self.side.norm, x)


class GosizenForCausalLM(nn.Module):
    has_request_state = True          # convolutions and recurrent layers remember a state per request: no prefix reuse
    residual_dtype = torch.float32

    def __init__(self, vllm_config: VllmConfig):
        super().__init__()
        mc = vllm_config.model_config
        cfg, dtype = mc.hf_config, mc.torch_dtype
        self.cfg, self.dtype = cfg, dtype
        if get_tensor_model_parallel_world_size() > 1 or get_pp_group().world_size > 1:
            raise NotImplementedError("Gosizen runs on one device: its norms reduce over whole rows and its recurrent "
                                      "state is not sharded")
        self.is_first = self.is_last = True
        width, eps = int(cfg["width"]), float((cfg.get("norm") or {}).get("eps", 1e-5))
        specs = cfg["layers"]
        if not specs:
            raise ValueError("a Gosizen model needs at least one layer")
        self.width, self.eps = width, eps
        self.start_layer, self.end_layer = 0, len(specs)
        self.loop = cfg.get("loop") or None
        self.runs = layer_runs(len(specs), self.loop)
        passes = [0] * len(specs)
        for r in self.runs:
            passes[r.layer] = max(passes[r.layer], r.index + 1)
        side_dim = int((cfg.get("token_side") or {}).get("dim") or 0)
        self.embed = VocabParallelEmbedding(int(cfg["vocab"]), width, dtype)
        self.side_embed = (nn.Parameter(torch.empty(int(cfg["vocab"]), side_dim * len(specs), dtype=dtype),
                                        requires_grad=False) if side_dim else None)
        if self.loop:
            self.loop_in = ReplicatedLinear(2 * width, width, False, dtype)
            self.loop_step = _f32(int(self.loop["times"]), width)
        from ..config import resolve_model_path
        from .loader import checkpoint_tensor_shapes
        shapes = {} if mc.load_format == "dummy" else checkpoint_tensor_shapes(resolve_model_path(mc.model))
        self.layers = nn.ModuleList(GosizenLayer(width, s, eps, i, dtype, passes[i], side_dim, shapes)
                                    for i, s in enumerate(specs))
        self.final_norm = ResidualRMSNorm(width, eps, dtype, offset=1.0)
        self.head = ColumnParallelLinear(width, [int(cfg["vocab"])], False, dtype)
        self.logit_softcap = float(cfg.get("logit_softcap") or 0.0)
        self.trace_residual: Optional[List[torch.Tensor]] = None      # tests: the residual stream after every run

    def rebind_buffers(self) -> None:
        return None

    def attention_layers(self) -> List[Attention]:
        """Every run's cache owner, in the order the runs execute."""
        out = []
        for r in self.runs:
            mix = self.layers[r.layer].mix
            out.append((mix.left if isinstance(mix, ParallelMixer) else mix).attn[r.index])
        return out

    def state_layers(self) -> List[SlotState]:
        out: List[SlotState] = []
        for r in self.runs:
            mix = self.layers[r.layer].mix
            if isinstance(mix, ParallelMixer):
                out += [mix.left.conv_states[r.index], mix.right.conv_states[r.index], mix.right.rule_states[r.index]]
        return out

    def decode_capturable(self) -> bool:
        return all(l.mlp.decode_capturable(self.dtype) for l in self.layers if isinstance(l.mlp, BiasedTopKMoE))

    def forward(self, input_ids, positions, intermediate: Optional[IntermediateTensors] = None):
        x = ops.embed_scaled(input_ids, self.embed.weight, 1.0)
        table = None if self.side_embed is None else self.side_embed.data
        x0 = self.embed(input_ids) if self.loop else None      # the embedding output, in the model dtype
        h = None                       # the next layer's normed input, or in front of a pass the stream itself
        n = len(self.runs)
        for r, run in enumerate(self.runs):
            layer = self.layers[run.layer]
            if run.opens >= 0:
                xb = x0 if h is None else h
                x = ops.linear_f32(torch.cat([xb, x0], dim=-1), self.loop_in.weight)
                x += self.loop_step[run.opens]
                h = None
            if h is None:
                h = layer.norm1(x)
            if r + 1 == n:
                then = self.final_norm
            else:
                then = None if self.runs[r + 1].opens >= 0 else self.layers[self.runs[r + 1].layer].norm1
            h = layer(x, h, run.index, input_ids, table, then)
            if self.trace_residual is not None:
                self.trace_residual.append(x.clone())
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        y = ops.linear_f32(hidden, self.head.weight)[..., :int(self.cfg["vocab"])]
        if self.logit_softcap > 0:
            y = torch.tanh(y / self.logit_softcap) * self.logit_softcap
        return y

    # ------------------------------------------------------------ weights
    _LATENT = {"dq": ("proj.weight", 0), "dkv": ("proj.weight", 1), "g": ("proj.weight", 2),
               "dq.norm": ("dq_norm", None), "dkv.norm": ("dkv_norm", None), "uq": ("uq.weight", None),
               "uk": ("uk", None), "uv": ("uv", None), "sink": ("sink", None), "o": ("o.weight", None)}
    _LEFT = {"q": ("left.proj.weight", 0), "k": ("left.proj.weight", 1), "v": ("left.proj.weight", 2),
             "g": ("left.proj.weight", 3), "q.b": ("left.proj.bias", 0), "k.b": ("left.proj.bias", 1),
             "v.b": ("left.proj.bias", 2), "q.conv": ("left.conv.weight", 0), "k.conv": ("left.conv.weight", 1),
             "v.conv": ("left.conv.weight", 2), "sink": ("left.sink", None), "o": ("o.weight", ("cols", 0))}
    _RIGHT = {"q": ("right.proj.weight", 0), "k": ("right.proj.weight", 1), "v": ("right.proj.weight", 2),
              "b": ("right.proj.weight", 3), "a1": ("right.proj.weight", 4), "g1": ("right.proj.weight", 5),
              "a2": ("right.a2.weight", None), "g2": ("right.g2.weight", None),
              "q.conv": ("right.conv.weight", 0), "k.conv": ("right.conv.weight", 1), "v.conv": ("right.conv.weight", 2),
              "A_log": ("right.rule.a_log", None), "dt_bias": ("right.rule.dt_bias", None),
              "norm": ("right.norm", None), "o": ("o.weight", ("cols", 1))}

    def _target(self, name: str):
        """Checkpoint tensor name -> (parameter name, shard of a fused parameter)."""
        top = {"embed": "embed.weight", "final.norm": "final_norm.weight", "head": "head.weight",
               "side.embed": "side_embed", "loop.in": "loop_in.weight", "loop.step": "loop_step"}
        if name in top:
            return top[name], None
        if not name.startswith("l"):
            return None
        idx, _, rest = name[1:].partition(".")
        if not idx.isdigit() or int(idx) >= len(self.layers):
            return None
        layer, base = self.layers[int(idx)], f"layers.{idx}."
        if rest == "norm1":
            return base + "norm1.weight", None
        kind, _, leaf = rest.partition(".")
        if kind == "side" and layer.side is not None:
            t = {"gate": "side.gate.weight", "proj": "side.proj.weight", "norm": "side.norm"}.get(leaf)
            return (base + t, None) if t else None
        if kind == "mix":
            if isinstance(layer.mix, GatedLatentMixer):
                table = self._LATENT
            else:
                half, _, leaf = leaf.partition(".")
                table = {"left": self._LEFT, "right": self._RIGHT}.get(half, {})
            if leaf not in table:
                return None
            p, shard = table[leaf]
            return base + "mix." + p, shard
        if kind != "mlp" or layer.mlp is None:
            return None
        if isinstance(layer.mlp, GeluMLP):
            return (base + f"mlp.{leaf}.weight", None) if leaf in ("up", "down") else None
        flat = {"router": "gate.weight", "router.b": "gate_bias"}
        if leaf in flat:
            return base + "mlp." + flat[leaf], None
        e, _, part = leaf.partition(".")
        if e[:1] == "e" and e[1:].isdigit() and int(e[1:]) < layer.mlp.num_experts and part in ("up", "down"):
            return base + ("mlp.w1" if part == "up" else "mlp.w2"), int(e[1:])
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
            if isinstance(shard, tuple):          # a run of columns of the fused output projection
                mix = self.layers[int(name[1:].partition(".")[0])].mix
                lo = 0 if shard[1] == 0 else mix.left.out_cols
                w = materialize(w)
                p.data[:, lo:lo + w.shape[1]].copy_(w)
                loaded.append(name)
                continue
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
    """Checkpoint tensor names and shapes of a Gosizen config (for the random-weight loader)."""
    width, vocab, n = int(c["width"]), int(c["vocab"]), len(c["layers"])
    out: Dict[str, Tuple[int, ...]] = {"embed": (vocab, width)}
    side = int((c.get("token_side") or {}).get("dim") or 0)
    if c.get("loop"):
        out["loop.in"], out["loop.step"] = (width, 2 * width), (int(c["loop"]["times"]), width)
    if side:
        out["side.embed"] = (vocab, side * n)
    for i, spec in enumerate(c["layers"]):
        m, p = spec["mixer"], f"l{i}."
        out[p + "norm1"] = (width,)
        if spec["type"] == "latent_attention":
            heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"])
            rank, rope, qr = int(m["kv_rank"]), int(m["rot_dim"]), int(m["q_rank"])
            q = p + "mix."
            out[q + "dq"], out[q + "dq.norm"], out[q + "uq"] = (qr, width), (qr,), (heads * (dim + rope), qr)
            out[q + "dkv"], out[q + "dkv.norm"] = (rank + rope, width), (rank,)
            out[q + "uk"], out[q + "uv"] = (heads * dim, rank), (heads * vdim, rank)
            out[q + "sink"], out[q + "g"], out[q + "o"] = (heads,), (heads, width), (width, heads * vdim)
        else:
            l, q = m["left"], p + "mix.left."
            heads, kvh, dim, vdim = int(l["heads"]), int(l.get("kv_heads") or l["heads"]), int(l["dim"]), int(l.get("vdim") or l["dim"])
            for nm, rows in (("q", heads * dim), ("k", kvh * dim), ("v", kvh * vdim)):
                out[q + nm], out[q + nm + ".b"], out[q + nm + ".conv"] = (rows, width), (rows,), (rows, int(l["conv"]))
            out[q + "sink"], out[q + "g"], out[q + "o"] = (heads,), (heads * vdim, width), (width, heads * vdim)
            r, q = m["right"], p + "mix.right."
            heads, kvh, dim, vdim = int(r["heads"]), int(r.get("kv_heads") or r["heads"]), int(r["dim"]), int(r.get("vdim") or r["dim"])
            for nm, rows in (("q", kvh * dim), ("k", kvh * dim), ("v", heads * vdim)):
                out[q + nm], out[q + nm + ".conv"] = (rows, width), (rows, int(r["conv"]))
            dr, gr = int(r["decay_rank"]), int(r["gate_rank"])
            out[q + "b"], out[q + "A_log"], out[q + "norm"] = (heads, width), (heads,), (vdim,)
            out[q + "a1"], out[q + "a2"], out[q + "dt_bias"] = (dr, width), (heads * dim, dr), (heads * dim,)
            out[q + "g1"], out[q + "g2"], out[q + "o"] = (gr, width), (heads * vdim, gr), (width, heads * vdim)
        mlp = spec.get("mlp")
        if mlp and mlp.get("kind", "dense") == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"] = (int(mlp["ff"]), width), (width, int(mlp["ff"]))
        elif mlp:
            ff = int(mlp["expert"]["ff"])
            for e in range(int(mlp["router"]["experts"])):
                out[f"{p}mlp.e{e}.up"], out[f"{p}mlp.e{e}.down"] = (ff, width), (width, ff)
            out[p + "mlp.router"], out[p + "mlp.router.b"] = (int(mlp["router"]["experts"]), width), (int(mlp["router"]["experts"]),)
        if side:
            out[p + "side.gate"], out[p + "side.proj"], out[p + "side.norm"] = (side, width), (width, side), (width,)
    out["final.norm"], out["head"] = (width,), (vocab, width)
    return out


def random_weight(name: str, shape: Tuple[int, ...], gen: torch.Generator, device, dtype) -> torch.Tensor:
    """A plausible random value for a checkpoint tensor (projections that keep the variance, stored norm weights
    around zero or one as the tensor asks, small biases, decays spread over (0, 1))."""
    def uni(lo: float, hi: float) -> torch.Tensor:
        return lo + (hi - lo) * torch.rand(shape, generator=gen, device=device, dtype=torch.float32)
    leaf = name.rsplit(".", 1)[-1]
    if leaf == "norm1" or name == "final.norm":
        w = uni(-0.2, 0.2)
    elif leaf == "norm":
        w = uni(0.8, 1.2)
    elif leaf in ("b", "sink", "dt_bias", "step") and len(shape) == 1 or name == "loop.step":
        w = uni(-0.5, 0.5)
    elif leaf == "A_log":
        w = uni(-1.0, 1.0)
    elif leaf == "conv":
        w = uni(-0.6, 0.6)
    elif name in ("embed", "side.embed"):
        w = uni(-1.0, 1.0)
    else:
        s = (3.0 / shape[-1]) ** 0.5
        w = uni(-s, s)
    return w.to(dtype)
