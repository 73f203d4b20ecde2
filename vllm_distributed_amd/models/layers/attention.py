"""Attention layer over the paged KV cache, plus the per-step forward context.

The model runner publishes one ``AttentionMetadata`` per step; every layer's
``Attention.forward`` reads it.  A batch is ordered decode-first: the first
``num_decodes`` sequences contribute one query token each and go to the
split-KV decode kernel; the rest (prompt chunks, possibly continuing a cached
prefix) go to the varlen prefill kernel.  Both read K/V through block tables.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn

from ... import ops


@dataclass
class AttentionMetadata:
    num_decodes: int                 # sequences with q_len == 1, at the front
    num_decode_tokens: int           # == num_decodes
    num_prefills: int
    num_prefill_tokens: int
    slot_mapping: torch.Tensor       # [T] int32 (cache slot per token, -1 = skip)
    block_table: torch.Tensor        # [B, max_blocks] int32
    seq_lens: torch.Tensor           # [B] int32 (context length incl. this step)
    query_start_loc: torch.Tensor    # [B+1] int32
    max_query_len: int
    max_seq_len: int
    # prefill-only views (sequence index rebased to the prefill part)
    prefill_query_start_loc: Optional[torch.Tensor] = None
    max_prefill_query_len: int = 0
    max_decode_seq_len: int = 0
    decode_workspace: Optional[torch.Tensor] = None
    # every prefill sequence of the step starts at position 0 (no cached context, no earlier chunk)
    prefill_fresh: bool = False
    # [B] int32: the slot of each sequence in per-request state tensors (layers with recurrent or convolution
    # state; the persistent batch's row), or None when the model keeps no such state
    state_slots: Optional[torch.Tensor] = None

    def token_rows(self, positions: torch.Tensor):
        """Per token of the step: the block-table row it reads (None = its own index: a pure decode batch)
        and the number of keys it sees (its position + 1).  For kernels whose rows are tokens
        (``LatentAttention``); computed once per step and kept."""
        if self.num_prefills == 0:
            return None, self.seq_lens
        cached = getattr(self, "_token_rows", None)
        if cached is None:
            t = positions.shape[0]
            idx = torch.arange(t, dtype=self.query_start_loc.dtype, device=positions.device)
            rows = torch.bucketize(idx, self.query_start_loc[1:], right=True).to(torch.int32)
            cached = self._token_rows = (rows, (positions + 1).to(torch.int32))
        return cached


def _prefill_token_rows(self, positions: torch.Tensor) -> torch.Tensor:
    """For the prompt-chunk rows of the step (those behind the decode rows): the sequence each belongs to, counted
    from the first prefill sequence; computed once per step and kept."""
    cached = getattr(self, "_prefill_rows", None)
    if cached is None:
        rows = self.token_rows(positions)[0]
        cached = self._prefill_rows = (rows[self.num_decode_tokens:] - self.num_decodes).contiguous()
    return cached


AttentionMetadata.prefill_token_rows = _prefill_token_rows


class ForwardContext:
    attn_metadata: Optional[AttentionMetadata] = None
    positions: Optional[torch.Tensor] = None


_CTX = ForwardContext()


def set_forward_context(attn_metadata: Optional[AttentionMetadata],
                        positions: Optional[torch.Tensor] = None) -> None:
    _CTX.attn_metadata = attn_metadata
    _CTX.positions = positions


def get_forward_context() -> ForwardContext:
    return _CTX


class Attention(nn.Module):
    """Owns one layer's slice of the KV cache (bound by the model runner)."""

    KERNEL_HEAD_DIMS = (64, 96, 128, 256)

    def __init__(self, num_heads: int, head_dim: int, num_kv_heads: int, scale: float,
                 layer_idx: int, sliding_window: Optional[int] = None, pad_head_dim: bool = False,
                 softcap: Optional[float] = None):
        super().__init__()
        # ``pad_head_dim`` (callers of ``forward`` only): a head size the attention kernels are not
        # built for (Phi-2's 80) is zero-padded to the next one they are; ``head_dim`` is then the
        # size q / k / v have in the cache and the kernels, ``model_head_dim`` the model's own.
        # Zero columns change neither the scores nor (sliced off again) the output.
        self.model_head_dim = head_dim
        if pad_head_dim and head_dim not in self.KERNEL_HEAD_DIMS and head_dim < self.KERNEL_HEAD_DIMS[-1]:
            head_dim = next(d for d in self.KERNEL_HEAD_DIMS if d > head_dim)
        self.num_heads, self.head_dim, self.num_kv_heads = num_heads, head_dim, num_kv_heads
        self.scale = scale
        # a query sees its last `window` keys only (0 = the whole context)
        self.window = int(sliding_window or 0)
        # scores squashed to softcap * tanh(score / softcap) before the softmax (Gemma-2); 0 = off
        self.softcap = float(softcap or 0.0)
        self.layer_idx = layer_idx
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None
        # e4m3 cache only: (k_scale[Hkv], v_scale[Hkv]) fp32; stored = value / scale.  None = 1.0
        self.kv_scales: Optional[tuple] = None
        # fp32 [num_heads] each, or None: an extra softmax column per head that is dropped after the softmax
        # (attention sinks: gpt-oss), and the slopes of a linear position bias (ALiBi: Bloom, MPT, Falcon-RW)
        self.sinks: Optional[torch.Tensor] = None
        self.alibi_slopes: Optional[torch.Tensor] = None

    def bind_kv_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_scales: Optional[tuple] = None) -> None:
        self.k_cache, self.v_cache, self.kv_scales = k_cache, v_cache, kv_scales

    def kv_cache_shapes(self, num_blocks: int, block_size: int):
        """Shapes of this layer's two cache tensors."""
        dims = (num_blocks, self.num_kv_heads, self.head_dim, block_size)
        return ops.k_cache_shape(*dims), ops.v_cache_shape(*dims)

    def kv_values_per_token(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim

    def set_kv_scale(self, which: str, value: torch.Tensor) -> None:
        """Checkpoint ``k_scale`` / ``v_scale`` (a scalar, or one value per local KV head)."""
        ks, vs = self.kv_scales or (None, None)
        t = value.detach().float().reshape(-1)
        t = (t.expand(self.num_kv_heads) if t.numel() == 1 else t).contiguous().clone()
        ones = torch.ones(self.num_kv_heads, dtype=torch.float32, device=t.device)
        ks, vs = (t, vs if vs is not None else ones) if which == "k" else (ks if ks is not None else ones, t)
        self.kv_scales = (ks, vs)

    def forward_cached(self, q: torch.Tensor) -> torch.Tensor:
        """``q[T, Hq*D]`` (already rotated; this step's K/V already in the cache)."""
        md = _CTX.attn_metadata
        t = q.shape[0]
        qv = q.view(t, self.num_heads, self.head_dim)
        if md is None:               # memory-profiling pass: no cache bound
            return q
        out = torch.empty((t, self.num_heads, self.head_dim), dtype=q.dtype, device=q.device)
        nd = md.num_decode_tokens
        if nd > 0:
            ops.paged_attention_decode(
                qv[:nd], self.k_cache, self.v_cache, md.block_table[:md.num_decodes],
                md.seq_lens[:md.num_decodes], self.scale, md.max_decode_seq_len,
                out=out[:nd], workspace=md.decode_workspace, kv_scales=self.kv_scales, window=self.window,
                softcap=self.softcap, sinks=self.sinks, alibi_slopes=self.alibi_slopes)
        if md.num_prefills > 0:
            ops.paged_attention(
                qv[nd:], self.k_cache, self.v_cache, md.block_table[md.num_decodes:],
                md.prefill_query_start_loc, md.seq_lens[md.num_decodes:], self.scale,
                md.max_prefill_query_len, md.max_seq_len, out=out[nd:], kv_scales=self.kv_scales,
                window=self.window, softcap=self.softcap, sinks=self.sinks, alibi_slopes=self.alibi_slopes)
        return out.view(t, self.num_heads * self.head_dim)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """Unfused path: write k/v (``[T, Hkv*D]``) to the cache, then attend."""
        md = _CTX.attn_metadata
        if self.head_dim != self.model_head_dim:
            t, extra = q.shape[0], self.head_dim - self.model_head_dim
            pad = torch.nn.functional.pad
            if md is None:
                return q
            k = pad(k.reshape(t, self.num_kv_heads, self.model_head_dim), (0, extra))
            v = pad(v.reshape(t, self.num_kv_heads, self.model_head_dim), (0, extra))
            ops.reshape_and_cache(k, v, self.k_cache, self.v_cache, md.slot_mapping, self.kv_scales)
            qp = pad(q.reshape(t, self.num_heads, self.model_head_dim), (0, extra))
            out = self.forward_cached(qp.view(t, self.num_heads * self.head_dim))
            return out.view(t, self.num_heads, self.head_dim)[..., :self.model_head_dim].reshape(
                t, self.num_heads * self.model_head_dim)
        if md is not None:
            t = k.shape[0]
            ops.reshape_and_cache(k.reshape(t, self.num_kv_heads, self.head_dim),
                                  v.reshape(t, self.num_kv_heads, self.head_dim),
                                  self.k_cache, self.v_cache, md.slot_mapping, self.kv_scales)
        return self.forward_cached(q)


class LatentAttention(Attention):
    """Multi-head latent attention with the up-projections absorbed into the query and the output: every head
    attends over ONE shared key ``[normalised c_kv | rotated k_rope]`` (``rank + rope`` wide) whose first ``rank``
    values are also the value.  The cache holds that row twice - as a key row and in the V^T fragment layout - so
    ``rank + rope + rank`` values per token where per-head keys and values would take ``heads * 2 * head_dim``."""
    latent = True

    def __init__(self, num_heads: int, rank: int, rope: int, scale: float, layer_idx: int):
        super().__init__(num_heads, rank + rope, 1, scale, layer_idx)
        self.v_dim = rank

    def kv_cache_shapes(self, num_blocks: int, block_size: int):
        return (ops.k_cache_shape(num_blocks, 1, self.head_dim, block_size),
                ops.v_cache_shape(num_blocks, 1, self.v_dim, block_size))

    def kv_values_per_token(self) -> int:
        return self.head_dim + self.v_dim

    def forward_latent(self, q: torch.Tensor, latent: torch.Tensor) -> torch.Tensor:
        """``q[T, H, rank + rope]`` (absorbed, rotated), ``latent[T, rank + rope]`` of this step's tokens:
        writes the cache, returns ``[T, H, rank]``."""
        md = _CTX.attn_metadata
        if md is None:                          # memory-profiling pass: no cache bound
            return q[..., :self.v_dim].contiguous()
        ops.mla_cache_write(latent, self.k_cache, self.v_cache, md.slot_mapping)
        return self.attend(q)

    def attend(self, q: torch.Tensor) -> torch.Tensor:
        """``q[T, H, rank + rope]`` against the cache (this step's rows already written) -> ``[T, H, rank]``."""
        md = _CTX.attn_metadata
        rows, lens = md.token_rows(_CTX.positions)
        return ops.mla_attention(q, self.k_cache, self.v_cache, md.block_table, rows, lens, self.scale, md.max_seq_len)


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict] = None):
    """Angular frequencies of a rotation over ``dims`` values paired half-apart, ``f_i = base^(-2i / dims)`` for
    ``i < dims / 2``, as an fp32 tensor, and the factor both cos and sin are multiplied by.  ``scaling`` =
    ``{factor, original, fast, slow}`` blends towards ``f_i / factor`` the YaRN way: with ``d(r) = dims *
    ln(original / (2 pi r)) / (2 ln base)`` the index at which a pair turns ``r`` times within ``original``
    positions, a ramp rises linearly from 0 at ``max(floor(d(fast)), 0)`` to 1 at ``min(ceil(d(slow)), dims - 1)``;
    pair ``i`` gets ``ramp_i f_i / factor + (1 - ramp_i) f_i``, and the factor is ``0.1 ln(factor) + 1``.
    ``scaling`` = ``{factor, original, low, high}`` slows by wavelength bands instead (Llama 3.1's rule): with
    ``l = 2 pi / f``, ``f`` stays where ``l < original / high``, becomes ``f / factor`` where ``l > original / low``,
    and between the two is ``(1 - s) f / factor + s f`` with ``s = (original / l - low) / (high - low)``; factor 1."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    scale = 1.0
    if scaling and "low" in scaling and "high" in scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])
        low, high = float(scaling["low"]), float(scaling["high"])
        wavelength = 2.0 * math.pi / f
        s = (original / wavelength - low) / (high - low)
        blended = (1.0 - s) * f / factor + s * f
        f = torch.where(wavelength < original / high, f, torch.where(wavelength > original / low, f / factor, blended))
    elif scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def index_of(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        scale = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32), float(scale)


class RowLatentAttention(Attention):
    """Latent attention over ONE row cache: a token's row is ``[normalised latent (rank) | rotated shared key part
    (rope)]``, its first ``rank`` values are also its value, and the per-head up-projections are folded into the
    query and the output by the caller.  Any ``rank`` / ``rope``; the rotation is computed from ``inv_freq`` in the
    kernel (positions and angles in fp32), so no table bounds the positions; scores, softmax and the weighted sum are
    fp32 in every dtype.  ``source``: another layer's instance whose rows this layer reads instead of keeping its own
    (layers that share keys and values: the reader allocates nothing and writes nothing).  ``window``: a query sees
    itself and the ``window - 1`` tokens before it (0: everything); ``sink``: a learned number per head whose
    exponential joins the softmax denominator (a parameter, or another instance's parameter to share);
    ``interleaved``: the rotation pairs neighbouring values instead of values half the rotated width apart."""
    latent = True
    row_cache = True

    def __init__(self, num_heads: int, rank: int, rope: int, scale: float, layer_idx: int,
                 source: Optional["RowLatentAttention"] = None, dtype: Optional[torch.dtype] = None,
                 window: int = 0, sink=False, interleaved: bool = False):
        super().__init__(num_heads, rank + rope, 1, scale, layer_idx, sliding_window=window)
        self.rank, self.rope, self.v_dim = rank, rope, rank
        self.interleaved = bool(interleaved)
        if isinstance(sink, nn.Parameter):
            self.sink = sink
        else:
            self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32), requires_grad=False) if sink else None
        # where the matrix-core latent kernel is built for this width and type, the values are cached once more as
        # its V^T fragments and it serves the layer (with fp32-precise softmax weights); else the plain kernel
        on_gpu = torch.empty(0).device.type != "cpu"       # (modules are built under the target device)
        self.fragments = bool(on_gpu and dtype is not None and rank % 16 == 0
                              and ops.mla_kernel_ok(rank + rope, rank, dtype))
        if source is not None:
            self.fragments = source.fragments
        if source is not None and (source.rank, source.rope) != (rank, rope):
            raise ValueError(f"layer {layer_idx} reads the latent rows of layer {source.layer_idx}, which have "
                             f"another shape ({source.rank} + {source.rope} against {rank} + {rope})")
        # (kept out of the module tree: the owner is registered where it lives)
        object.__setattr__(self, "source", source)

    def kv_cache_shapes(self, num_blocks: int, block_size: int):
        if self.fragments:
            return (num_blocks, 1, block_size, self.head_dim), ops.v_cache_shape(num_blocks, 1, self.rank, block_size)
        return (num_blocks, 1, block_size, self.head_dim), (num_blocks, 0)

    def kv_values_per_token(self) -> int:
        return self.head_dim + (self.rank if self.fragments else 0)

    def bind_kv_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_scales: Optional[tuple] = None) -> None:
        if k_cache.dtype == torch.float8_e4m3fn:
            raise ValueError("an e4m3 KV cache is not supported for latent rows read in the model dtype; "
                             "use --kv-cache-dtype auto")
        super().bind_kv_cache(k_cache, v_cache, kv_scales)

    @property
    def rows(self) -> Optional[torch.Tensor]:
        return (self.source if self.source is not None else self).k_cache

    def forward_latent(self, q: torch.Tensor, nope: int, q_lat: torch.Tensor, latent: Optional[torch.Tensor],
                       norm_weight: Optional[torch.Tensor], eps: float, inv_freq: torch.Tensor,
                       rot_scale: float, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``q[T, H, nope + rope]``, ``q_lat[H, T, rank]``, ``latent[T, rank + rope]`` (None for a reader of another
        layer's rows): norm, rotations, cache write and query assembly in one op, then attention -> ``[T, H, rank]``;
        ``gate[T, H]`` (raw): head ``h``'s result times ``sigmoid(gate[t, h])``."""
        md, pos = _CTX.attn_metadata, _CTX.positions
        write = latent is not None and self.source is None and md is not None
        qf = ops.latent_prep(q, nope, q_lat, latent if write else None, norm_weight, eps, inv_freq, rot_scale, pos,
                             self.k_cache if write else None, md.slot_mapping if write else None,
                             self.v_cache if write and self.fragments else None, self.interleaved)
        if md is None:                          # memory-profiling pass: no cache bound
            return qf[..., :self.rank].contiguous()
        rows, lens = md.token_rows(pos)
        if self.fragments:
            owner = self.source if self.source is not None else self
            return ops.mla_attention(qf, owner.k_cache, owner.v_cache, md.block_table, rows, lens, self.scale,
                                     md.max_seq_len, precise=True, window=self.window, sinks=self.sink, gate=gate)
        return ops.latent_row_attention(qf, self.rows, md.block_table, rows, lens, self.scale, self.rank, md.max_seq_len,
                                        self.window, self.sink, gate)


class WindowBiasAttention(Attention):
    """Attention whose window keeps the first keys of the sequence, with a logarithmic distance bias instead of
    a rotation, an optional score cap, a sink in the softmax denominator and a sigmoid gate on each head's output;
    key and value heads may differ in size.  A query at position ``i`` sees key ``j <= i`` when
    ``i - j < window`` or ``j < keep_first``; its score is ``cap(q.k * scale) - bias_scale[h] * ln(1 +
    bias_rate[h] * (i - j))``.  The caches are key rows ``[blocks, Hkv, block, dim]`` and values with eight keys side
    by side per channel, ``[blocks, Hkv, block / 8, vdim, 8]``, written by ``ops.conv_norm_cache`` (this layer's callers convolve and normalise q / k / v
    first); scores, softmax and the weighted sum of values are fp32 in every dtype.  ``chunk > 0`` replaces the window
    by blocks of ``chunk`` positions counted from the sequence's start: a query sees the keys of its own block up to
    itself (``window`` is then ``chunk``: no key further back is ever read, so the pages behind it are given back).
    ``sink`` may be another instance's parameter (layers that run several times over one set of weights)."""
    row_cache = True

    def __init__(self, num_heads: int, dim: int, vdim: int, num_kv_heads: int, scale: float, layer_idx: int,
                 window: int = 0, keep_first: int = 0, softcap: Optional[float] = None, distance_bias: bool = True,
                 sink=True, chunk: int = 0):
        self.chunk = int(chunk or 0)
        if self.chunk:
            window, keep_first = self.chunk, 0
        super().__init__(num_heads, dim, num_kv_heads, scale, layer_idx, sliding_window=window, softcap=softcap)
        self.vdim = vdim
        self.keep_first = int(keep_first or 0) if self.window else 0
        f32 = torch.float32
        # (fp32 whatever the model dtype: they enter the scores directly)
        self.bias_scale = nn.Parameter(torch.zeros(num_heads, dtype=f32), requires_grad=False) if distance_bias else None
        self.bias_rate = nn.Parameter(torch.zeros(num_heads, dtype=f32), requires_grad=False) if distance_bias else None
        if isinstance(sink, nn.Parameter):
            self.sink = sink
        else:
            self.sink = nn.Parameter(torch.zeros(num_heads, dtype=f32), requires_grad=False) if sink else None

    def kv_cache_shapes(self, num_blocks: int, block_size: int):
        if block_size % 8:
            raise ValueError("block_size must be a multiple of 8")
        return ((num_blocks, self.num_kv_heads, block_size, self.head_dim),
                (num_blocks, self.num_kv_heads, block_size // 8, self.vdim, 8))

    def kv_values_per_token(self) -> int:
        return self.num_kv_heads * (self.head_dim + self.vdim)

    def bind_kv_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_scales: Optional[tuple] = None) -> None:
        if k_cache.dtype == torch.float8_e4m3fn:
            raise ValueError("an e4m3 KV cache is not supported for attention over convolved, normalised keys "
                             "(its kernels read the cache in the model dtype); use --kv-cache-dtype auto")
        super().bind_kv_cache(k_cache, v_cache, kv_scales)

    def forward_cached(self, q: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``q[T, Hq, dim]`` (this step's keys and values already cached), ``gate[T, Hq]`` raw -> ``[T, Hq * vdim]``."""
        md = _CTX.attn_metadata
        t = q.shape[0]
        if md is None:               # memory-profiling pass: no cache bound
            return q.new_zeros((t, self.num_heads * self.vdim))
        out = torch.empty((t, self.num_heads, self.vdim), dtype=q.dtype, device=q.device)
        pos = _CTX.positions
        nd, nb = md.num_decode_tokens, md.num_decodes
        common = (self.scale, self.softcap, self.window, self.keep_first, self.bias_scale, self.bias_rate, self.sink)
        if nd > 0:            # one row per sequence: the waves of a block share its keys
            ops.window_bias_attention(q[:nd], self.k_cache, self.v_cache, md.block_table[:nb], md.query_start_loc[:nb + 1],
                                      md.seq_lens[:nb], None, pos[:nd], *common,
                                      None if gate is None else gate[:nd], 1, out=out[:nd], chunk=self.chunk)
        if md.num_prefills > 0:
            ops.window_bias_attention(q[nd:], self.k_cache, self.v_cache, md.block_table[nb:],
                                      md.prefill_query_start_loc, md.seq_lens[nb:], md.prefill_token_rows(pos), pos[nd:],
                                      *common, None if gate is None else gate[nd:], md.max_prefill_query_len,
                                      out=out[nd:], chunk=self.chunk)
        return out.view(t, self.num_heads * self.vdim)


class CrossedBiasAttention(WindowBiasAttention):
    """Causal softmax attention with the logarithmic distance bias of ``WindowBiasAttention`` whose VALUES ARE ITS
    KEYS before their norm (the key rows hold the normed keys, the values the projection itself, so ``vdim = dim`` and
    there is no value projection) and whose heads exchange their softmax weights: ``weight_h <- sum_g talk[h, g]
    weight_g``, each head then reading the values of the key / value head it belongs to with its mixed weights.  Computed as
    ``o_h = sum_g talk[h, g] * (weight_g applied to the values of h's key / value head)``: the attention kernel
    applies every query head's weights to every value head (fp32 ``[T, H, Hkv, dim]``) and ``ops.mix_heads`` sums.
    Callers norm q / k and write the cache with ``ops.joint_norm_cache``."""

    def __init__(self, num_heads: int, dim: int, num_kv_heads: int, scale: float, layer_idx: int,
                 distance_bias: bool = True):
        super().__init__(num_heads, dim, dim, num_kv_heads, scale, layer_idx, distance_bias=distance_bias, sink=False)
        self.talk = nn.Parameter(torch.eye(num_heads, dtype=torch.float32), requires_grad=False)

    def forward_cached(self, q: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``q[T, Hq, dim]`` (this step's keys and values already cached) -> ``[T, Hq * dim]`` in ``q``'s dtype."""
        md = _CTX.attn_metadata
        t = q.shape[0]
        if md is None:               # memory-profiling pass: no cache bound
            return q.new_zeros((t, self.num_heads * self.vdim))
        out = torch.empty((t, self.num_heads, self.num_kv_heads, self.vdim), dtype=torch.float32, device=q.device)
        pos = _CTX.positions
        nd, nb = md.num_decode_tokens, md.num_decodes
        common = (self.scale, self.bias_scale, self.bias_rate)
        if nd > 0:
            ops.crossed_bias_attention(q[:nd], self.k_cache, self.v_cache, md.block_table[:nb],
                                       md.query_start_loc[:nb + 1], md.seq_lens[:nb], None, pos[:nd], *common, 1,
                                       out=out[:nd])
        if md.num_prefills > 0:
            ops.crossed_bias_attention(q[nd:], self.k_cache, self.v_cache, md.block_table[nb:],
                                       md.prefill_query_start_loc, md.seq_lens[nb:], md.prefill_token_rows(pos),
                                       pos[nd:], *common, md.max_prefill_query_len, out=out[nd:])
        return ops.mix_heads(out, self.talk, q.dtype)


class ScalarRMSNorm(nn.Module):
    """RMS norm whose gain is a single number for all coordinates, in fp32 arithmetic; ``forward`` returns the
    model dtype (the input of a projection), ``residual_add`` folds a sublayer's output into the fp32 residual
    stream through this norm and hands back the next sublayer's normed input in the same launch."""

    def __init__(self, eps: float, dtype: torch.dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.ones((), dtype=torch.float32), requires_grad=False)
        self.eps, self.dtype = eps, dtype

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.scalar_rms_norm(x, self.weight, self.eps, out_dtype or self.dtype)

    def residual_add(self, y: torch.Tensor, residual: torch.Tensor, then: Optional["ScalarRMSNorm"] = None):
        return ops.scalar_norm_residual(y, self.weight, residual, None if then is None else then.weight, self.eps,
                                        self.dtype)


class ResidualRMSNorm(nn.Module):
    """RMS norm over an fp32 residual stream in fp32 arithmetic, with fp32 gains ``offset + weight`` (``offset`` 1: the
    checkpoint keeps the gain minus one).  ``forward`` returns the model dtype (the input of a projection); ``add`` folds one or
    two sublayer outputs into the stream and hands back the normed sum in the same launch; ``after`` does so for an
    output that is itself RMS-normed with ``post_weight`` before it joins the stream."""

    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, offset: float = 0.0):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(hidden_size, dtype=torch.float32), requires_grad=False)
        self.eps, self.dtype, self.offset = eps, dtype, float(offset)

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.rms_norm_to(x, self.weight, self.eps, out_dtype or self.dtype, self.offset)

    def add(self, residual: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.add_rms_norm_to(residual, a, b, self.weight, self.eps, self.dtype, self.offset)

    def after(self, y: torch.Tensor, post_weight: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        return ops.norm_add_norm(y, post_weight, residual, self.weight, self.eps, self.dtype, self.offset)


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype), requires_grad=False)
        self.eps = eps

    def forward(self, x, residual: Optional[torch.Tensor] = None):
        """``x`` may be a value its producer left unfinished - a projection's K-split partial sums
        (``layers.linear.PartialSums``) or the expert rows of a sparse block before their weighted sum
        (``layers.moe.ExpertRows``): with a residual, the kernel that adds and normalises finishes it."""
        if not isinstance(x, torch.Tensor):
            if residual is not None:
                return x.add_rms_norm(residual, self.weight, self.eps)
            x = x.materialize()
        if residual is None:
            return ops.rms_norm(x, self.weight, self.eps)
        return ops.fused_add_rms_norm(x, residual, self.weight, self.eps)


class LayerNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, bias: bool = True):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=dtype), requires_grad=False) if bias else None
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layer_norm(x, self.weight, self.bias, self.eps)


class ResidualLayerNorm(nn.Module):
    """Layer norm with weight and bias over an fp32 residual stream, in fp32 arithmetic (parameters kept in fp32);
    ``forward`` returns the model dtype (the input of a projection), ``add`` folds a sublayer's output into the
    stream and hands back the normed sum in the same launch."""

    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, bias: bool = True):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float32), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=torch.float32), requires_grad=False) if bias else None
        self.eps, self.dtype = eps, dtype

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.layer_norm_to(x, self.weight, self.bias, self.eps, out_dtype or self.dtype)

    def add(self, y: torch.Tensor, residual: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.add_layer_norm(y, residual, self.weight, self.bias, self.eps, out_dtype or self.dtype)
