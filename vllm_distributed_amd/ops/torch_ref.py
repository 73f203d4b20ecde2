"""Plain-PyTorch implementations of every op in ``ops``.

They define the semantics (the HIP kernels are tested against these in fp32)
and are the execution path on CPU.  KV-cache layouts are the ones the CDNA4
kernels consume as MFMA operands straight from global memory:

* ``k_cache[num_blocks, num_kv_heads, block_size, head_dim]``  - a key row is
  contiguous in ``head_dim`` (the QK^T reduction axis);
* ``v_cache[num_blocks, num_kv_heads, head_dim // 16, block_size // 8, 16, 8]``  -
  V^T in MFMA-fragment order: the 8 keys of one ``head_dim`` row are a 16-byte
  chunk (the PV reduction axis), 16 rows of a key group are adjacent, and the
  key groups of a block follow each other inside a 16-row slab.  A wave's
  16-row x 32-key fragment is one contiguous 1 KiB run, and a decode step's new
  token lands in ``head_dim / 16`` runs of 256 bytes per head instead of one
  element in each of ``head_dim`` separate rows.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F


# ------------------------------------------------------------------- norms
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (y * weight.float()).to(x.dtype)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                       eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """``r = x + residual``; returns ``(rms_norm(r), r)`` (r rounded to x.dtype
    before the norm, as the fused kernel stores it)."""
    r = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(r, weight, eps), r


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               eps: float) -> torch.Tensor:
    return F.layer_norm(x.float(), (x.shape[-1],), weight.float(),
                        None if bias is None else bias.float(), eps).to(x.dtype)


# -------------------------------------------------------------- activation
def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    return (F.silu(x[..., :d].float()) * x[..., d:].float()).to(x.dtype)


# ------------------------------------------------------------------ rotary
def build_cos_sin_cache(head_dim: int, max_pos: int, theta: float,
                        rope_scaling: Optional[dict] = None,
                        rotary_dim: Optional[int] = None) -> torch.Tensor:
    """``[max_pos, rotary_dim]`` fp32: cos in the first half, sin in the second."""
    rd = rotary_dim or head_dim
    inv_freq = 1.0 / (theta ** (torch.arange(0, rd, 2, dtype=torch.float64) / rd))
    if rope_scaling:
        rtype = rope_scaling.get("rope_type", rope_scaling.get("type"))
        if rtype == "llama3":
            factor = rope_scaling.get("factor", 8.0)
            lo = rope_scaling.get("low_freq_factor", 1.0)
            hi = rope_scaling.get("high_freq_factor", 4.0)
            old = rope_scaling.get("original_max_position_embeddings", 8192)
            wavelen = 2 * math.pi / inv_freq
            smooth = ((old / wavelen) - lo) / (hi - lo)
            scaled = torch.where(wavelen > old / lo, inv_freq / factor,
                                 torch.where(wavelen < old / hi, inv_freq,
                                             (1 - smooth) * inv_freq / factor + smooth * inv_freq))
            inv_freq = scaled
        elif rtype == "linear":
            inv_freq = inv_freq / rope_scaling.get("factor", 1.0)
        elif rtype == "dynamic":
            # NTK-aware base stretch, fixed for the configured context (the table is built once)
            factor = rope_scaling.get("factor", 1.0)
            old = rope_scaling.get("original_max_position_embeddings") or max_pos
            if max_pos > old:
                base = theta * ((factor * max_pos / old) - (factor - 1)) ** (rd / (rd - 2))
                inv_freq = 1.0 / (base ** (torch.arange(0, rd, 2, dtype=torch.float64) / rd))
        elif rtype == "yarn":
            # interpolate the low-frequency dims by `factor`, keep the high-frequency
            # ones, blend linearly in between; cos/sin carry the attention temperature
            factor = float(rope_scaling.get("factor", 1.0))
            old = rope_scaling.get("original_max_position_embeddings") or max_pos
            beta_fast = float(rope_scaling.get("beta_fast") or 32)
            beta_slow = float(rope_scaling.get("beta_slow") or 1)

            def corr_dim(rot: float) -> float:
                return rd * math.log(old / (rot * 2 * math.pi)) / (2 * math.log(theta))
            low = max(math.floor(corr_dim(beta_fast)), 0)
            high = min(math.ceil(corr_dim(beta_slow)), rd - 1)
            if rope_scaling.get("truncate") is False:
                low, high = max(corr_dim(beta_fast), 0), min(corr_dim(beta_slow), rd - 1)
            ramp = ((torch.arange(rd // 2, dtype=torch.float64) - low) / max(high - low, 1e-3)).clamp(0, 1)
            keep = 1.0 - ramp
            inv_freq = inv_freq / factor * (1 - keep) + inv_freq * keep
            mscale = rope_scaling.get("attention_factor")
            if mscale is None:
                ms, ms_all = rope_scaling.get("mscale"), rope_scaling.get("mscale_all_dim")

                def get_mscale(scale: float, m: float = 1.0) -> float:
                    return 1.0 if scale <= 1 else 0.1 * m * math.log(scale) + 1.0
                mscale = get_mscale(factor, ms) / get_mscale(factor, ms_all) if ms and ms_all else get_mscale(factor)
            t = torch.arange(max_pos, dtype=torch.float64)
            freqs = torch.outer(t, inv_freq)
            return (torch.cat([freqs.cos(), freqs.sin()], dim=-1) * float(mscale)).float()
        elif rtype in ("longrope", "su"):
            # LongRoPE: one divisor per frequency, a "short" set for sequences inside the original context and a
            # "long" one beyond it, and a temperature on cos / sin.  transformers switches sets when a sequence
            # grows past the original context (its cached keys keep the other rotation); here the table is built
            # once for the served context: the long set throughout when ``max_pos`` exceeds the original context,
            # the short one otherwise - what a sequence longer / shorter than that gets there.
            old = int(rope_scaling.get("original_max_position_embeddings") or max_pos)
            full = int(rope_scaling.get("max_position_embeddings") or max_pos)
            factor = float(rope_scaling.get("factor") or full / old)
            which = "long_factor" if max_pos > old else "short_factor"
            if not rope_scaling.get(which):
                raise ValueError(f"LongRoPE scaling needs short_factor and long_factor lists ({which} is missing)")
            ext = rope_scaling[which]
            if len(ext) != rd // 2:
                raise ValueError(f"LongRoPE lists {len(ext)} factors for {rd // 2} frequencies")
            inv_freq = inv_freq / torch.tensor(ext, dtype=torch.float64)
            mscale = rope_scaling.get("attention_factor")
            if mscale is None:
                mscale = 1.0 if factor <= 1.0 else math.sqrt(1 + math.log(factor) / math.log(old))
            t = torch.arange(max_pos, dtype=torch.float64)
            freqs = torch.outer(t, inv_freq)
            return (torch.cat([freqs.cos(), freqs.sin()], dim=-1) * float(mscale)).float()
        elif rtype not in (None, "default"):
            raise ValueError(f"rope scaling type {rtype!r} is not supported")
    t = torch.arange(max_pos, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()


def rotary_embedding(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                     cos_sin_cache: torch.Tensor, head_dim: int) -> None:
    """NeoX-style rotation in place on ``q[T, Hq*D]`` and ``k[T, Hkv*D]``."""
    rd = cos_sin_cache.shape[-1]
    cs = cos_sin_cache.index_select(0, positions.long())
    cos, sin = cs[:, :rd // 2].unsqueeze(1), cs[:, rd // 2:].unsqueeze(1)
    for t in (q, k):
        v = t.view(t.shape[0], -1, head_dim)
        x1 = v[..., :rd // 2].float()
        x2 = v[..., rd // 2:rd].float()
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        v[..., :rd // 2] = o1.to(t.dtype)
        v[..., rd // 2:rd] = o2.to(t.dtype)


# ---------------------------------------------------------------- KV cache
FP8_KV = torch.float8_e4m3fn
FP8_MAX = 448.0
V_GROUP = 8          # keys per contiguous chunk of the V cache
V_ROWS = 16          # head_dim rows per slab (the M of one MFMA fragment)


def v_cache_shape(num_blocks: int, num_kv_heads: int, head_dim: int, block_size: int) -> Tuple[int, ...]:
    if block_size % V_GROUP != 0:
        raise ValueError(f"block_size must be a multiple of {V_GROUP}")
    if head_dim % V_ROWS != 0:
        raise ValueError(f"head_dim must be a multiple of {V_ROWS}")
    return (num_blocks, num_kv_heads, head_dim // V_ROWS, block_size // V_GROUP, V_ROWS, V_GROUP)


def k_cache_shape(num_blocks: int, num_kv_heads: int, head_dim: int, block_size: int) -> Tuple[int, ...]:
    return (num_blocks, num_kv_heads, block_size, head_dim)


def _to_cache(x: torch.Tensor, cache: torch.Tensor, scale: Optional[torch.Tensor]) -> torch.Tensor:
    """``x[T, Hkv, D]`` in the cache's element type; an e4m3 cache stores ``x / scale[head]``, saturated."""
    if cache.dtype != FP8_KV:
        return x.to(cache.dtype)
    xf = x.float()
    if scale is not None:
        xf = xf / scale.float().view(1, -1, 1)
    return xf.clamp_(-FP8_MAX, FP8_MAX).to(FP8_KV)


def reshape_and_cache(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, slot_mapping: torch.Tensor, kv_scales=None) -> None:
    """Scatter ``k,v[T, Hkv, D]`` into the paged caches; slot < 0 is skipped."""
    bs = k_cache.shape[2]
    valid = slot_mapping >= 0
    slots = slot_mapping[valid].long()
    blk, off = slots // bs, slots % bs
    ks, vs = kv_scales if kv_scales is not None else (None, None)
    if k_cache.dtype == FP8_KV:      # index assignment is not implemented for 8-bit floats: go through the bytes
        k_cache.view(torch.uint8)[blk, :, off, :] = _to_cache(k[valid], k_cache, ks).view(torch.uint8)
        vv = _to_cache(v[valid], v_cache, vs).view(torch.uint8)
        v_cache.view(torch.uint8)[blk, :, :, off // V_GROUP, :, off % V_GROUP] = vv.unflatten(-1, (-1, V_ROWS))
        return
    k_cache[blk, :, off, :] = k[valid].to(k_cache.dtype)
    v_cache[blk, :, :, off // V_GROUP, :, off % V_GROUP] = v[valid].to(v_cache.dtype).unflatten(-1, (-1, V_ROWS))


def rope_and_cache(positions: torch.Tensor, qkv: torch.Tensor, cos_sin_cache: torch.Tensor,
                   k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                   num_heads: int, num_kv_heads: int, head_dim: int, q_norm_weight=None, k_norm_weight=None,
                   norm_eps: float = 0.0, kv_scales=None) -> torch.Tensor:
    """Rotate q and k inside the packed ``qkv[T, (Hq+2Hkv)*D]``, write k/v to
    the cache, return the rotated ``q[T, Hq*D]`` (a view of qkv).  With norm
    weights each q and k head is RMS-normalised first."""
    qs, ks = num_heads * head_dim, num_kv_heads * head_dim
    q, k, v = qkv[:, :qs], qkv[:, qs:qs + ks], qkv[:, qs + ks:]
    if q_norm_weight is not None:
        for part, w in ((q, q_norm_weight), (k, k_norm_weight)):
            h = part.reshape(part.shape[0], -1, head_dim).float()
            h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + norm_eps) * w.float()
            part.copy_(h.reshape(part.shape).to(part.dtype))
    rotary_embedding(positions, q, k, cos_sin_cache, head_dim)
    reshape_and_cache(k.reshape(-1, num_kv_heads, head_dim), v.reshape(-1, num_kv_heads, head_dim),
                      k_cache, v_cache, slot_mapping, kv_scales)
    return q


def alibi_slopes(num_heads: int, kind: str = "bloom", bias_max: float = 8.0) -> torch.Tensor:
    """Per-head slopes of the linear position bias (fp32 ``[num_heads]``).  ``bloom`` (also Falcon-RW):
    a geometric sequence over the largest power of two not above the head count, the remaining heads
    taking every other step of the next finer sequence.  ``mpt``: the sequence over the next power of
    two at or above the head count with exponent step ``bias_max / n``, odd entries first when the
    count is not a power of two."""
    if kind == "mpt":
        n = 2 ** math.ceil(math.log2(num_heads))
        s = 1.0 / torch.pow(2.0, torch.arange(1, n + 1, dtype=torch.float32) * (bias_max / n))
        if n != num_heads:
            s = torch.cat([s[1::2], s[::2]])[:num_heads]
        return s.contiguous()
    n = 2 ** math.floor(math.log2(num_heads))
    base = 2.0 ** (-(2.0 ** -(math.log2(n) - 3)))
    s = torch.pow(torch.tensor(base, dtype=torch.float32), torch.arange(1, n + 1, dtype=torch.float32))
    if n != num_heads:
        extra = 2.0 ** (-(2.0 ** -(math.log2(2 * n) - 3)))
        rest = min(n, num_heads - n)
        s = torch.cat([s, torch.pow(torch.tensor(extra, dtype=torch.float32),
                                    torch.arange(1, 1 + 2 * rest, 2, dtype=torch.float32))])
    return s.contiguous()


def _gather_kv(k_cache, v_cache, block_table_row, seq_len, kv_scales=None):
    bs = k_cache.shape[2]
    nb = (seq_len + bs - 1) // bs
    blocks = block_table_row[:nb].long()
    if k_cache.dtype == FP8_KV:
        k = k_cache.view(torch.uint8)[blocks].view(FP8_KV).float()
        v = v_cache.view(torch.uint8)[blocks].view(FP8_KV).float()
        if kv_scales is not None:
            k = k * kv_scales[0].float().view(1, -1, 1, 1)
            v = v * kv_scales[1].float().view(1, -1, 1, 1, 1, 1)
    else:
        k = k_cache[blocks]                   # [nb, H, bs, D]
        v = v_cache[blocks]                   # [nb, H, D/16, bs/8, 16, 8]
    k = k.permute(1, 0, 2, 3).reshape(k.shape[1], nb * bs, -1)[:, :seq_len]
    v = v.permute(1, 0, 3, 5, 2, 4).reshape(v.shape[1], nb * bs, -1)[:, :seq_len]
    return k, v                               # [H, S, D]


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, query_start_loc: torch.Tensor,
                    seq_lens: torch.Tensor, scale: float, kv_scales=None, window: int = 0,
                    softcap: float = 0.0, sinks=None, alibi_slopes=None) -> torch.Tensor:
    """Causal attention of each sequence's query chunk against its paged KV
    (which already contains the chunk).  ``q[T, Hq, D]``; sequence ``i`` owns
    query rows ``query_start_loc[i]:query_start_loc[i+1]`` which are the last
    ``q_len`` positions of its ``seq_lens[i]`` tokens.  ``window > 0``: a query at
    position ``p`` sees keys ``p - window + 1 .. p`` only (sliding-window attention).
    ``softcap > 0``: scores are squashed to ``softcap * tanh(score / softcap)`` (Gemma-2).
    ``sinks [Hq]``: one extra score per head that joins the softmax and is then dropped (attention sinks).
    ``alibi_slopes [Hq]``: ``slope * (key position - query position)`` is added to the scores."""
    out = torch.empty_like(q)
    hq = q.shape[1]
    hkv = k_cache.shape[1]
    g = hq // hkv
    qsl = query_start_loc.tolist()
    sls = seq_lens.tolist()
    for i, sl in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        ql = e - s
        if ql == 0:
            continue
        k, v = _gather_kv(k_cache, v_cache, block_table[i], sl, kv_scales)
        k = k.float().repeat_interleave(g, dim=0)
        v = v.float().repeat_interleave(g, dim=0)
        qi = q[s:e].float().transpose(0, 1)                     # [Hq, ql, D]
        scores = torch.matmul(qi, k.transpose(1, 2)) * scale    # [Hq, ql, sl]
        if softcap > 0:
            scores = torch.tanh(scores / softcap) * softcap
        qpos = torch.arange(sl - ql, sl, device=q.device).unsqueeze(1)
        kpos = torch.arange(sl, device=q.device).unsqueeze(0)
        if alibi_slopes is not None:
            scores = scores + alibi_slopes.float().view(-1, 1, 1) * (kpos - qpos).float()
        scores = scores.masked_fill(kpos > qpos, float("-inf"))
        if window > 0:
            scores = scores.masked_fill(kpos <= qpos - window, float("-inf"))
        if sinks is not None:
            col = sinks.float().view(-1, 1, 1).expand(hq, ql, 1)
            probs = torch.softmax(torch.cat([scores, col], dim=-1), -1)[..., :-1]
        else:
            probs = torch.softmax(scores, -1)
        out[s:e] = torch.matmul(probs, v).transpose(0, 1).to(q.dtype)
    return out


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_table: torch.Tensor, seq_lens: torch.Tensor,
                           scale: float, kv_scales=None, window: int = 0, softcap: float = 0.0,
                           sinks=None, alibi_slopes=None) -> torch.Tensor:
    b = q.shape[0]
    qsl = torch.arange(b + 1, device=q.device, dtype=torch.int32)
    return paged_attention(q, k_cache, v_cache, block_table, qsl, seq_lens, scale, kv_scales, window, softcap,
                           sinks, alibi_slopes)


# ---------------------------------------------------------------- sampling
def apply_penalties(logits: torch.Tensor, token_counts: torch.Tensor, prompt_mask: torch.Tensor,
                    presence: torch.Tensor, frequency: torch.Tensor,
                    repetition: torch.Tensor) -> torch.Tensor:
    """``token_counts[B,V]`` = occurrences in the output so far;
    ``prompt_mask[B,V]`` = token appears in the prompt."""
    seen = (token_counts > 0) | prompt_mask
    rep = repetition.unsqueeze(1)
    logits = torch.where(seen, torch.where(logits > 0, logits / rep, logits * rep), logits)
    logits = logits - frequency.unsqueeze(1) * token_counts
    logits = logits - presence.unsqueeze(1) * (token_counts > 0)
    return logits


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, min_p: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    """One token per row.  ``temperature == 0`` rows are argmax.  ``uniform[B]``
    in (0,1) drives inverse-CDF sampling over the *descending-sorted* filtered
    distribution, so an identical ``uniform`` gives identical tokens on every
    implementation."""
    logits = logits.float()
    greedy = temperature == 0
    t = torch.where(greedy, torch.ones_like(temperature), temperature)
    probs = torch.softmax(logits / t.unsqueeze(1), dim=-1)
    sp, si = probs.sort(dim=-1, descending=True, stable=True)
    v = logits.shape[-1]
    ranks = torch.arange(v, device=logits.device).unsqueeze(0)
    k = torch.where(top_k <= 0, torch.full_like(top_k, v), top_k).unsqueeze(1)
    keep = ranks < k
    cum = sp.cumsum(-1)
    keep &= (cum - sp) < top_p.unsqueeze(1)          # keep until mass reaches top_p
    keep &= sp >= (min_p.unsqueeze(1) * sp[:, :1])
    keep[:, 0] = True
    sp = torch.where(keep, sp, torch.zeros_like(sp))
    total = sp.sum(-1, keepdim=True)
    cdf = sp.cumsum(-1)
    target = uniform.unsqueeze(1).to(cdf.dtype) * total
    idx = (cdf < target).sum(-1).clamp(max=v - 1)
    # guard: never pick a filtered-out entry because of rounding at the tail
    n_keep = keep.sum(-1)
    idx = torch.minimum(idx, n_keep - 1)
    sampled = si.gather(1, idx.unsqueeze(1)).squeeze(1)
    return torch.where(greedy, logits.argmax(-1), sampled)


def compute_logprobs(logits: torch.Tensor, token_ids: torch.Tensor, num_top: int):
    lp = torch.log_softmax(logits.float(), dim=-1)
    chosen = lp.gather(1, token_ids.unsqueeze(1).long()).squeeze(1)
    if num_top > 0:
        tv, ti = lp.topk(num_top, dim=-1)
    else:
        tv = ti = None
    return chosen, tv, ti


def embedding(ids: torch.Tensor, weight: torch.Tensor, vocab_start: int = 0,
              masked: bool = False) -> torch.Tensor:
    """Vocab-parallel gather: ids outside ``[vocab_start, vocab_start+rows)``
    produce zero rows (summed across ranks afterwards)."""
    local = ids.long() - vocab_start
    mask = (local >= 0) & (local < weight.shape[0])
    out = F.embedding(torch.where(mask, local, torch.zeros_like(local)), weight)
    if masked or vocab_start != 0:
        out = out * mask.unsqueeze(-1).to(out.dtype)
    return out


# ------------------------------------------------ multi-head latent attention over a latent cache (DeepSeek)
def mla_cache_write(latent: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    slot_mapping: torch.Tensor) -> None:
    """``latent[T, DK]`` into ``k_cache[blocks, 1, bs, DK]``; its first DV values into the V^T fragment cache."""
    bs = k_cache.shape[2]
    dv = v_cache.shape[2] * V_ROWS
    valid = slot_mapping[:latent.shape[0]] >= 0
    slots = slot_mapping[:latent.shape[0]][valid].long()
    blk, off = slots // bs, slots % bs
    if k_cache.dtype == FP8_KV:      # e4m3 cache, scale 1, saturating; index assignment goes through the bytes
        x = latent[valid].float().clamp_(-FP8_MAX, FP8_MAX).to(FP8_KV).view(torch.uint8)
        k_cache.view(torch.uint8)[blk, 0, off, :] = x
        v_cache.view(torch.uint8)[blk, 0, :, off // V_GROUP, :, off % V_GROUP] = x[:, :dv].unflatten(-1, (-1, V_ROWS))
        return
    x = latent[valid].to(k_cache.dtype)
    k_cache[blk, 0, off, :] = x
    v_cache[blk, 0, :, off // V_GROUP, :, off % V_GROUP] = x[:, :dv].unflatten(-1, (-1, V_ROWS))


def mla_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                  token_seq: Optional[torch.Tensor], seq_lens: torch.Tensor, scale: float, max_seq_len: int = 0,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``q[T, Hq, DK]`` against the latent cache -> ``[T, Hq, DV]`` in fp32 arithmetic.  Keys come from the
    key-row cache, values from the V^T fragment cache (so a test of a kernel against this checks both)."""
    t, hq, dk = q.shape
    bs = k_cache.shape[2]
    dv = v_cache.shape[2] * V_ROWS
    res = torch.zeros((t, hq, dv), dtype=torch.float32, device=q.device)
    rows = token_seq.long() if token_seq is not None else torch.arange(t, device=q.device)
    lens = seq_lens[:t].long()
    for b in torch.unique(rows).tolist():
        mine = torch.nonzero(rows == b).flatten()
        n = int(lens[mine].max())
        blocks = block_table[b, :(n + bs - 1) // bs].long()
        kb, vb = k_cache, v_cache
        if k_cache.dtype == FP8_KV:
            kb, vb = k_cache.view(torch.uint8), v_cache.view(torch.uint8)
        keys = kb[blocks, 0].reshape(-1, dk)[:n]
        # [blocks, DV/16, bs/8, 16, 8] -> [blocks, bs/8, 8, DV/16, 16] -> [n, DV]
        vals = vb[blocks, 0].permute(0, 2, 4, 1, 3).reshape(-1, dv)[:n]
        if k_cache.dtype == FP8_KV:
            keys, vals = keys.contiguous().view(FP8_KV), vals.contiguous().view(FP8_KV)
        keys, vals = keys.float(), vals.float()
        s = torch.einsum("thd,nd->thn", q[mine].float(), keys) * scale
        mask = torch.arange(n, device=q.device)[None, None, :] >= lens[mine][:, None, None]
        p = torch.softmax(s.masked_fill(mask, float("-inf")), dim=-1)
        res[mine] = torch.einsum("thn,nd->thd", p, vals)
    res = res.to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


# ------------------------------------------------ single-gain RMS norms, PolyNorm, short convolutions with state
def scalar_rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * gain`` with one gain for the whole row, in fp32 arithmetic."""
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * gain.float()
    return y.to(out_dtype)


def scalar_norm_residual(y: torch.Tensor, post_gain: torch.Tensor, residual: torch.Tensor,
                         next_gain: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype):
    """``residual += norm(y) * post_gain`` in place on the fp32 residual stream; with ``next_gain`` also returns
    ``norm(residual) * next_gain`` (the input of the sublayer that follows) in ``out_dtype``."""
    residual.add_(scalar_rms_norm(y, post_gain, eps, torch.float32))
    if next_gain is None:
        return None
    return scalar_rms_norm(residual, next_gain, eps, out_dtype)


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """``c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3`` with element-wise powers and ``N(u) = u / sqrt(mean(u^2) + eps)``
    over the last dimension; fp32 arithmetic, result in ``z``'s dtype."""
    zf = z.float()
    c = coef.float()
    out = torch.full_like(zf, float(c[3]))
    p = zf
    for i in range(3):
        out = out + c[i] * p * torch.rsqrt(p.pow(2).mean(-1, keepdim=True) + eps)
        p = p * zf
    return out.to(z.dtype)


def short_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, slots: torch.Tensor,
               query_start_loc: torch.Tensor, seq_lens: torch.Tensor) -> torch.Tensor:
    """Causal per-channel convolution over time of the packed rows ``x[T, C]`` with tap-major ``weight[taps, C]``:
    ``y_t = sum_j weight[j] * u_(t - taps + 1 + j)``, zero before a sequence's first position.  Sequence ``i``
    owns rows ``query_start_loc[i]:query_start_loc[i+1]``, the last positions of its ``seq_lens[i]`` tokens; the
    ``taps - 1`` inputs in front of them come from ``state[slots[i]]`` (``[slots, taps - 1, C]``, oldest first),
    which is left holding the last ``taps - 1`` inputs of the sequence.  Returns fp32 ``[T, C]``."""
    taps = weight.shape[0]
    r = taps - 1
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    wf = weight.float()
    qsl, sls, sl = query_start_loc.tolist(), seq_lens.tolist(), slots.tolist()
    for i, n_ctx in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        n = e - s
        if n == 0:
            continue
        start = n_ctx - n
        hist = state[sl[i]].float() if r else x.new_zeros((0, x.shape[1]), dtype=torch.float32)
        if start < r:                      # positions before the sequence's start read as zero, whatever the slot held
            hist = hist.clone()
            hist[:r - start] = 0
        u = torch.cat([hist, x[s:e].float()], 0)
        acc = torch.zeros((n, x.shape[1]), dtype=torch.float32, device=x.device)
        for j in range(taps):
            acc += wf[j] * u[j:j + n]
        y[s:e] = acc
        if r:
            state[sl[i]] = u[u.shape[0] - r:].to(state.dtype)
    return y


def conv_norm_cache(x: torch.Tensor, conv_weight: torch.Tensor, state: torch.Tensor, slots: torch.Tensor,
                    query_start_loc: torch.Tensor, seq_lens: torch.Tensor, num_heads: int, num_kv_heads: int,
                    dim: int, vdim: int, q_norm: torch.Tensor, k_norm: torch.Tensor, eps: float,
                    v_first: Optional[torch.Tensor], v_lambda: Optional[torch.Tensor], keep_v: bool,
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], slot_mapping: torch.Tensor,
                    inv_freq: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None):
    """Everything between the fused projection and the attention of a layer whose q / k / v pass through a short
    convolution: ``x[T, C_x]`` holds ``[q | k | v | ...]`` (columns past the three are not touched);
    ``short_conv`` over the first ``C`` columns, RMS norm of each q and k head with the ``[dim]`` weights (skipped when
    ``q_norm`` is None), then, with ``inv_freq``, the rotation of each q and k head's first ``2 * len(inv_freq)``
    values by ``positions`` (value ``i`` paired with value ``i + len(inv_freq)``),
    ``v <- (1 - v_lambda) v + v_lambda v_first`` when ``v_first[T, Hkv * vdim]`` (fp32) is given, k and the mixed
    v into the row caches ``[blocks, Hkv, block, dim | vdim]`` at ``slot_mapping``.  Returns ``(q[T, Hq, dim]``
    in ``x``'s dtype, the unmixed fp32 ``v`` if ``keep_v`` else None``)``."""
    t = x.shape[0]
    qs, ks, vs = num_heads * dim, num_kv_heads * dim, num_kv_heads * vdim
    c = qs + ks + vs
    y = short_conv(x[:, :c], conv_weight, state, slots, query_start_loc, seq_lens)

    def head_norm(u, w):
        if w is None:
            return u
        return u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()

    q = head_norm(y[:, :qs].reshape(t, num_heads, dim), q_norm)
    k = head_norm(y[:, qs:qs + ks].reshape(t, num_kv_heads, dim), k_norm)
    if inv_freq is not None and inv_freq.numel():
        q = rotate_pairs_first(q, positions[:t], inv_freq, 1.0)
        k = rotate_pairs_first(k, positions[:t], inv_freq, 1.0)
    q = q.to(x.dtype)
    v = y[:, qs + ks:].reshape(t, num_kv_heads, vdim)
    kept = v.reshape(t, vs).clone() if keep_v else None
    if v_first is not None:
        lam = v_lambda.float()
        v = (1.0 - lam) * v + lam * v_first.reshape(t, num_kv_heads, vdim)
    if k_cache is not None:
        bs = k_cache.shape[2]
        valid = slot_mapping[:t] >= 0
        sm = slot_mapping[:t][valid].long()
        blk, off = sm // bs, sm % bs
        k_cache[blk, :, off, :] = k[valid].to(k_cache.dtype)
        v_cache[blk, :, off // V_GROUP, :, off % V_GROUP] = v[valid].to(v_cache.dtype)
    return q, kept


def window_bias_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                          query_start_loc: torch.Tensor, seq_lens: torch.Tensor, scale: float, softcap: float,
                          window: int, keep_first: int, bias_scale: Optional[torch.Tensor],
                          bias_rate: Optional[torch.Tensor], sinks: Optional[torch.Tensor],
                          gate: Optional[torch.Tensor], chunk: int = 0) -> torch.Tensor:
    """Causal attention over ``k_cache[blocks, Hkv, block, D]`` (key rows) and ``v_cache[blocks, Hkv, block / 8, Dv,
    8]`` (eight keys side by side per channel).
    A query at position ``i`` sees key ``j <= i`` when ``i - j < window`` (``window`` 0: no limit) or
    ``j < keep_first``; with ``chunk > 0`` it sees ``j <= i`` only inside its own block of ``chunk`` positions
    counted from the sequence's start (``i // chunk == j // chunk``).  ``score = q.k * scale``, squashed to ``softcap * tanh(score / softcap)`` when
    ``softcap > 0``, minus ``bias_scale[h] * ln(1 + bias_rate[h] * (i - j))``; ``sinks[h]`` adds ``exp(sinks[h])``
    to the softmax denominator; ``gate[T, Hq]`` multiplies head ``h``'s output by ``sigmoid(gate[t, h])``.
    fp32 arithmetic; returns ``[T, Hq, Dv]`` in ``q``'s dtype."""
    t, hq, d = q.shape
    hkv, bs, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    g = hq // hkv
    out = torch.zeros((t, hq, dv), dtype=torch.float32, device=q.device)
    qsl, sls = query_start_loc.tolist(), seq_lens.tolist()
    for i, sl in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        ql = e - s
        if ql == 0:
            continue
        blocks = block_table[i, :(sl + bs - 1) // bs].long()
        k = k_cache[blocks].permute(1, 0, 2, 3).reshape(hkv, -1, d)[:, :sl].float().repeat_interleave(g, dim=0)
        v = v_cache[blocks].permute(1, 0, 2, 4, 3).reshape(hkv, -1, dv)[:, :sl].float().repeat_interleave(g, dim=0)
        qi = q[s:e].float().transpose(0, 1)
        sc = torch.matmul(qi, k.transpose(1, 2)) * scale
        if softcap > 0:
            sc = torch.tanh(sc / softcap) * softcap
        qpos = torch.arange(sl - ql, sl, device=q.device).unsqueeze(1)
        kpos = torch.arange(sl, device=q.device).unsqueeze(0)
        dist = (qpos - kpos).clamp(min=0).float()
        if bias_scale is not None:
            sc = sc - bias_scale.float().view(-1, 1, 1) * torch.log1p(bias_rate.float().view(-1, 1, 1) * dist)
        seen = kpos <= qpos
        if window > 0:
            seen = seen & (((qpos - kpos) < window) | (kpos < keep_first))
        if chunk > 0:
            seen = seen & (torch.div(qpos, chunk, rounding_mode="floor") == torch.div(kpos, chunk, rounding_mode="floor"))
        sc = sc.masked_fill(~seen, float("-inf"))
        if sinks is not None:
            col = sinks.float().view(-1, 1, 1).expand(hq, ql, 1)
            p = torch.softmax(torch.cat([sc, col], dim=-1), -1)[..., :-1]
        else:
            p = torch.softmax(sc, -1)
        out[s:e] = torch.matmul(p, v).transpose(0, 1)
    if gate is not None:
        out = out * torch.sigmoid(gate.float()).unsqueeze(-1)
    return out.to(q.dtype)


# ------------------------------------------------ fp32 residual stream with layer norms, decayed linear attention,
# ------------------------------------------------ gated norm, clamped GLU, latent attention over one row cache
def embed_scaled(ids: torch.Tensor, weight: torch.Tensor, scale: float) -> torch.Tensor:
    """``weight[ids] * scale`` as the fp32 residual stream."""
    return weight[ids.long()].float() * scale


def layer_norm_to(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """Layer norm (mean taken off, biased variance, weight and bias) in fp32 arithmetic, result in ``out_dtype``."""
    xf = x.float()
    d = xf - xf.mean(-1, keepdim=True)
    y = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype)


def add_layer_norm(y: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                   eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``residual += y`` in place on the fp32 residual stream, then ``layer_norm_to`` of the sum."""
    residual.add_(y.float())
    return layer_norm_to(residual, weight, bias, eps, out_dtype)


def decay_linear_attention(x: torch.Tensor, num_heads: int, dim: int, vdim: int, decay: torch.Tensor,
                           state: torch.Tensor, slots: torch.Tensor, query_start_loc: torch.Tensor,
                           seq_lens: torch.Tensor, silu: bool = True) -> torch.Tensor:
    """Linear attention with one decay per head over the packed rows ``x[T, C]`` whose leading columns are
    ``[q (H * dim) | k (H * dim) | v (H * vdim)]`` (``silu``: each passed through SiLU first).  Per head
    ``S_t = decay[h] S_(t-1) + k_t v_t^T`` and ``o_t = S_t^T q_t``; ``S`` is ``state[slots[i]]`` (``[slots, H, dim,
    vdim]`` fp32) for sequence ``i``, taken as zero when the rows start at position 0 whatever the slot held, and left
    holding the state after the sequence's last row.  fp32 arithmetic; returns fp32 ``[T, H * vdim]``."""
    t = x.shape[0]
    h = num_heads
    qs, vs = h * dim, h * vdim
    xf = x[:, :2 * qs + vs].float()
    if silu:
        xf = F.silu(xf)
    q = xf[:, :qs].reshape(t, h, dim)
    k = xf[:, qs:2 * qs].reshape(t, h, dim)
    v = xf[:, 2 * qs:].reshape(t, h, vdim)
    out = torch.zeros((t, h, vdim), dtype=torch.float32, device=x.device)
    d = decay.float().view(h, 1, 1)
    qsl, sls, sl = query_start_loc.tolist(), seq_lens.tolist(), slots.tolist()
    for i, n_ctx in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        if e == s:
            continue
        st = state[sl[i]].float().clone() if n_ctx - (e - s) > 0 else torch.zeros_like(state[sl[i]], dtype=torch.float32)
        for r in range(s, e):
            st = d * st + k[r].unsqueeze(2) * v[r].unsqueeze(1)
            out[r] = torch.einsum("hkv,hk->hv", st, q[r])
        state[sl[i]] = st.to(state.dtype)
    return out.reshape(t, vs)


def gated_rms_norm(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, eps: float,
                   out_dtype: torch.dtype, group: int = 0, scale: float = 1.0,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``o / sqrt(mean(o^2) + eps) * weight * sigmoid(gate) * scale`` in fp32 arithmetic, the mean over whole rows or,
    with ``group > 0``, over each run of ``group`` values (``weight[group]`` then serves every run).  ``out``: a
    ``[T, N]`` view (rows may be strided) that receives the result."""
    of = o.float()
    if group > 0:
        g = of.unflatten(-1, (-1, group))
        y = (g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).flatten(-2)
    else:
        y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    y = y * torch.sigmoid(gate.float()) * scale
    if out is not None:
        out.copy_(y)
        return out
    return y.to(out_dtype)


def clamped_glu(h: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """``g sigmoid(alpha g) (u + 1)`` for ``h = [gate | up]`` with ``g = min(gate, limit)``, ``u = clamp(up, -limit,
    limit)``; fp32 arithmetic, result in ``h``'s dtype."""
    f = h.shape[-1] // 2
    g = h[..., :f].float().clamp(max=limit)
    u = h[..., f:].float().clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(h.dtype)


def rotate_half_first(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rot_scale: float) -> torch.Tensor:
    """Rotate the first ``2 * len(inv_freq)`` values of the last dimension of fp32 ``x[T, ..., n]``, value ``i``
    paired with value ``i + len(inv_freq)``, by the angle ``positions[t] * inv_freq[i]`` (fp32), cos and sin both
    times ``rot_scale``; the rest passes unchanged."""
    half = inv_freq.numel()
    a = positions.float().view(-1, *([1] * (x.dim() - 1))) * inv_freq.float()
    cos, sin = torch.cos(a) * rot_scale, torch.sin(a) * rot_scale
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., 2 * half:]], dim=-1)


def rotate_pairs_first(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rot_scale: float,
                       interleaved: bool = False) -> torch.Tensor:
    """``rotate_half_first`` with a choice of pairing: ``interleaved`` pairs value ``2i`` with value ``2i + 1``."""
    if not interleaved:
        return rotate_half_first(x.float(), positions, inv_freq, rot_scale)
    half = inv_freq.numel()
    xf = x.float()
    a = positions.float().view(-1, *([1] * (x.dim() - 1))) * inv_freq.float()
    cos, sin = torch.cos(a) * rot_scale, torch.sin(a) * rot_scale
    u, v = xf[..., 0:2 * half:2], xf[..., 1:2 * half:2]
    rot = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).flatten(-2)
    return torch.cat([rot, xf[..., 2 * half:]], dim=-1)


def latent_prep(q: torch.Tensor, nope: int, q_lat: torch.Tensor, latent: Optional[torch.Tensor],
                norm_weight: Optional[torch.Tensor], eps: float, inv_freq: torch.Tensor, rot_scale: float,
                positions: torch.Tensor, cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor],
                fragments: Optional[torch.Tensor] = None, interleaved: bool = False) -> torch.Tensor:
    """Between the projections and the attention of a layer whose keys and values are one shared latent row per
    token.  ``q[T, H, nope + rope]``, ``q_lat[H, T, rank]`` (the unrotated query part already multiplied into the
    latent space): returns ``[T, H, rank + rope] = [q_lat | rotated q[..., nope:]]``.  With ``latent[T, rank + rope]``
    the row ``[RMS norm of the first rank values * norm_weight | rotated last rope values]`` goes into
    ``cache[blocks, 1, block, rank + rope]`` at ``slot_mapping`` (a layer that reads another layer's rows passes
    None), and its first ``rank`` values also into ``fragments`` (the V^T fragment cache, see ``v_cache_shape``) when
    the layer keeps one.  Norm and rotation in fp32; ``interleaved`` pairs neighbouring values in the rotation."""
    t = q.shape[0]
    q_rot = rotate_pairs_first(q[..., nope:], positions[:t], inv_freq, rot_scale, interleaved)
    out = torch.cat([q_lat.transpose(0, 1).float(), q_rot], dim=-1).to(q.dtype)
    if latent is not None and cache is not None and slot_mapping is not None:
        rank = q_lat.shape[2]
        c = latent[:, :rank].float()
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_weight.float()
        kr = rotate_pairs_first(latent[:, rank:], positions[:t], inv_freq, rot_scale, interleaved)
        row = torch.cat([c, kr], dim=-1).to(cache.dtype)
        bs = cache.shape[2]
        valid = slot_mapping[:t] >= 0
        sm = slot_mapping[:t][valid].long()
        cache[sm // bs, 0, sm % bs, :] = row[valid]
        if fragments is not None and fragments.numel():       # the values once more, as V^T fragments
            off = sm % bs
            fragments[sm // bs, 0, :, off // V_GROUP, :, off % V_GROUP] = row[valid][:, :rank].unflatten(-1, (-1, V_ROWS))
    return out


def latent_row_attention(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
                         token_seq: Optional[torch.Tensor], seq_lens: torch.Tensor, scale: float, rank: int,
                         window: int = 0, sinks: Optional[torch.Tensor] = None,
                         gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``q[T, H, DK]`` against ``cache[blocks, 1, block, DK]``: token ``t`` reads block-table row ``token_seq[t]``
    (``t`` itself when None) and sees keys ``0 .. seq_lens[t] - 1``, with ``window > 0`` only the last ``window`` of
    them; a key row's first ``rank`` values are also its value.  ``sinks[H]`` adds ``exp(sinks[h])`` to head ``h``'s
    softmax denominator; ``gate[T, H]`` multiplies head ``h``'s output by ``sigmoid(gate[t, h])``.  Scores, softmax and
    the weighted sum in fp32; returns ``[T, H, rank]`` in ``q``'s dtype."""
    t, hq, dk = q.shape
    bs = cache.shape[2]
    res = torch.zeros((t, hq, rank), dtype=torch.float32, device=q.device)
    rows = token_seq[:t].long() if token_seq is not None else torch.arange(t, device=q.device)
    lens = seq_lens[:t].long()
    for b in torch.unique(rows).tolist():
        mine = torch.nonzero(rows == b).flatten()
        n = int(lens[mine].max())
        if n == 0:
            continue
        first = max(int(lens[mine].min()) - window, 0) if window > 0 else 0      # (blocks before it may be gone)
        blocks = block_table[b, first // bs:(n + bs - 1) // bs].long()
        keys = cache[blocks, 0].reshape(-1, dk)[:n - first // bs * bs].float()
        kpos = torch.arange(first // bs * bs, n, device=q.device)[None, None, :]
        s = torch.einsum("thd,nd->thn", q[mine].float(), keys) * scale
        mask = kpos >= lens[mine][:, None, None]
        if window > 0:
            mask = mask | (kpos < lens[mine][:, None, None] - window)
        s = s.masked_fill(mask, float("-inf"))
        if sinks is not None:
            col = sinks.float().view(1, hq, 1).expand(mine.numel(), hq, 1)
            p = torch.softmax(torch.cat([s, col], dim=-1), dim=-1)[..., :-1]
        else:
            p = torch.softmax(s, dim=-1)
        res[mine] = torch.einsum("thn,nd->thd", p, keys[:, :rank])
    if gate is not None:
        res = res * torch.sigmoid(gate[:t].float()).unsqueeze(-1)
    return res.to(q.dtype)


def expert_epilogue(routed: torch.Tensor, x: torch.Tensor, topw: Optional[torch.Tensor], topi: Optional[torch.Tensor],
                    real_experts: int, shared: Optional[torch.Tensor], gate: Optional[torch.Tensor]) -> torch.Tensor:
    """``routed + x * s + shared * sigmoid(gate)`` with ``s`` the sum, per row, of the weights ``topw`` whose output
    ``topi`` is an identity expert (``>= real_experts``); ``gate`` one value per row.  fp32 arithmetic, result in
    ``routed``'s dtype."""
    out = routed.float()
    if topw is not None:
        out = out + x.float() * (topw.float() * (topi >= real_experts)).sum(-1, keepdim=True)
    if shared is not None:
        out = out + shared.float() * torch.sigmoid(gate.float().reshape(-1, 1))
    return out.to(routed.dtype)


# ------------------------------------------------ fp32 residual stream with offset RMS norms, side inputs per token,
# ------------------------------------------------ convolutions with activation, the gated delta rule
def rms_norm_to(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
                offset: float = 0.0) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * (offset + weight)`` over the last dimension in fp32 arithmetic (``weight`` None:
    no gain), result in ``out_dtype``."""
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * (weight.float() + offset)
    return y.to(out_dtype)


def add_rms_norm_to(residual: torch.Tensor, a: Optional[torch.Tensor], b: Optional[torch.Tensor],
                    weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype, offset: float = 0.0,
                    normed: bool = True) -> torch.Tensor:
    """``residual += a + b`` in place on the fp32 residual stream (either may be None), then ``rms_norm_to`` of the
    sum, or with ``normed`` False just the sum, in ``out_dtype``."""
    if a is not None:
        residual.add_(a.float() if b is None else a.float() + b.float())
    if not normed:
        return residual.to(out_dtype)
    return rms_norm_to(residual, weight, eps, out_dtype, offset)


def norm_add_norm(y: torch.Tensor, post_weight: torch.Tensor, residual: torch.Tensor,
                  next_weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype, next_offset: float = 0.0,
                  next_normed: bool = True) -> Optional[torch.Tensor]:
    """``residual += rms_norm(y) * post_weight`` in place on the fp32 residual stream; then what
    ``add_rms_norm_to(residual, None, None, next_weight, ...)`` returns."""
    residual.add_(rms_norm_to(y, post_weight, eps, torch.float32))
    if not next_normed:
        return residual.to(out_dtype)
    return rms_norm_to(residual, next_weight, eps, out_dtype, next_offset)


def gelu_tanh_f(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))


def gelu_mul_rows(g: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col: int) -> torch.Tensor:
    """``gelu_tanh(g[T, n]) * table[ids, col : col + n]`` in fp32 arithmetic, result in ``g``'s dtype."""
    n = g.shape[1]
    return (gelu_tanh_f(g.float()) * table[ids.long(), col:col + n].float()).to(g.dtype)


def sigmoid_mul(o: torch.Tensor, gate: torch.Tensor, scale: float = 1.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``o * sigmoid(gate) * scale`` in fp32 arithmetic, in ``o``'s dtype; ``out``: a view that receives it."""
    y = o.float() * torch.sigmoid(gate.float()) * scale
    if out is not None:
        out.copy_(y)
        return out
    return y.to(o.dtype)


def short_conv_act(x: torch.Tensor, channels: int, conv_weight: torch.Tensor, state: torch.Tensor, slots: torch.Tensor,
                   query_start_loc: torch.Tensor, seq_lens: torch.Tensor, silu: bool,
                   bias: Optional[torch.Tensor] = None, residual: bool = False) -> torch.Tensor:
    """``short_conv`` over the first ``channels`` columns of ``x`` (the state moves on), plus ``bias[channels]``,
    through SiLU when ``silu``; with ``residual`` the input itself is added at the end (``x + conv(x)``);
    ``[T, channels]`` in ``x``'s dtype."""
    y = short_conv(x[:, :channels], conv_weight, state, slots, query_start_loc, seq_lens)
    if bias is not None:
        y = y + bias.float()
    if silu:
        y = F.silu(y)
    if residual:
        y = y + x[:, :channels].float()
    return y.to(x.dtype)


def gated_delta_rule(x: torch.Tensor, num_heads: int, num_qk_heads: int, dim: int, vdim: int, beta: torch.Tensor,
                     dt: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, state: torch.Tensor,
                     slots: torch.Tensor, query_start_loc: torch.Tensor, seq_lens: torch.Tensor,
                     norm_eps: float = 1e-6) -> torch.Tensor:
    """The gated delta rule over the packed rows ``x[T, C]`` = ``[q (Hqk * dim) | k (Hqk * dim) | v (H * vdim)]``;
    value head ``h`` reads q / k head ``h // (H / Hqk)``.  Per row: q and k become unit vectors
    (``u / sqrt(sum(u^2) + norm_eps)``), q times ``dim^-0.5``; ``b = sigmoid(beta[t, h])``; one decay per head and
    key channel ``g = exp(-exp(a_log[h]) * softplus(dt[t, h, :] + dt_bias[h, :]))``; then ``S <- g * S`` by rows,
    ``u = b (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``.  ``S`` is ``state[slots[i]]`` (``[slots, H, dim, vdim]``
    fp32) for sequence ``i``, taken as zero when the rows start at position 0 whatever the slot held, and left holding
    the state after the sequence's last row.  fp32 arithmetic; returns fp32 ``[T, H * vdim]``."""
    t, h, g = x.shape[0], num_heads, num_qk_heads
    qs = g * dim
    xf = x[:, :2 * qs + h * vdim].float()
    q = xf[:, :qs].reshape(t, g, dim)
    k = xf[:, qs:2 * qs].reshape(t, g, dim)
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + norm_eps) * dim ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + norm_eps)
    q, k = q.repeat_interleave(h // g, dim=1), k.repeat_interleave(h // g, dim=1)
    v = xf[:, 2 * qs:].reshape(t, h, vdim)
    b = torch.sigmoid(beta[:t].float())
    decay = torch.exp(-torch.exp(a_log.float()).view(1, h, 1)
                      * F.softplus(dt[:t].float().reshape(t, h, dim) + dt_bias.float().view(1, h, dim)))
    out = torch.zeros((t, h, vdim), dtype=torch.float32, device=x.device)
    qsl, sls, sl = query_start_loc.tolist(), seq_lens.tolist(), slots.tolist()
    for i, n_ctx in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        if e == s:
            continue
        st = state[sl[i]].float().clone() if n_ctx - (e - s) > 0 else torch.zeros_like(state[sl[i]], dtype=torch.float32)
        for r in range(s, e):
            st = decay[r].unsqueeze(2) * st
            u = b[r].unsqueeze(1) * (v[r] - torch.einsum("hkv,hk->hv", st, k[r]))
            st = st + k[r].unsqueeze(2) * u.unsqueeze(1)
            out[r] = torch.einsum("hkv,hk->hv", st, q[r])
        state[sl[i]] = st.to(state.dtype)
    return out.reshape(t, h * vdim)


# ------------------------------------------------ selective state-space scan, gate in front of a grouped norm,
# ------------------------------------------------ q / k normed over all heads with values = keys, crossed value
# ------------------------------------------------ heads and mixed head weights
def selective_scan(x: torch.Tensor, dt: torch.Tensor, num_heads: int, groups: int, vdim: int, n_state: int,
                   a_log: torch.Tensor, dt_bias: torch.Tensor, d_skip: Optional[torch.Tensor], state: torch.Tensor,
                   slots: torch.Tensor, query_start_loc: torch.Tensor, seq_lens: torch.Tensor) -> torch.Tensor:
    """A state-space recurrence with one data-dependent decay per head over the packed rows ``x[T, C]`` =
    ``[u (H * vdim) | B (G * N) | C (G * N)]``; head ``h`` reads B / C group ``h // (H / G)``.  Per row
    ``d = softplus(dt[t, h] + dt_bias[h])`` (unbounded above), ``S <- exp(-exp(a_log[h]) * d) * S + d * B u^T`` (``S`` is
    ``N x vdim``), ``y = S^T C + d_skip[h] * u``.  ``S`` is ``state[slots[i]]`` (``[slots, H, N, vdim]`` fp32) for
    sequence ``i``, taken as zero when the rows start at position 0 whatever the slot held, and left holding the state
    after the sequence's last row.  fp32 arithmetic; returns fp32 ``[T, H * vdim]``."""
    t, h, g, n = x.shape[0], num_heads, groups, n_state
    inner = h * vdim
    xf = x[:, :inner + 2 * g * n].float()
    u = xf[:, :inner].reshape(t, h, vdim)
    bm = xf[:, inner:inner + g * n].reshape(t, g, n).repeat_interleave(h // g, dim=1)
    cm = xf[:, inner + g * n:].reshape(t, g, n).repeat_interleave(h // g, dim=1)
    d = F.softplus(dt[:t].float() + dt_bias.float().view(1, h), threshold=30.0)
    decay = torch.exp(-torch.exp(a_log.float()).view(1, h) * d)
    out = torch.zeros((t, h, vdim), dtype=torch.float32, device=x.device)
    qsl, sls, sl = query_start_loc.tolist(), seq_lens.tolist(), slots.tolist()
    for i, n_ctx in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        if e == s:
            continue
        st = state[sl[i]].float().clone() if n_ctx - (e - s) > 0 else torch.zeros_like(state[sl[i]], dtype=torch.float32)
        for r in range(s, e):
            st = decay[r].view(h, 1, 1) * st + (d[r].view(h, 1) * bm[r]).unsqueeze(2) * u[r].unsqueeze(1)
            out[r] = torch.einsum("hnv,hn->hv", st, cm[r])
        state[sl[i]] = st.to(state.dtype)
    if d_skip is not None:
        out = out + d_skip.float().view(1, h, 1) * u
    return out.reshape(t, inner)


def act_gate_group_norm(y: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, group: int,
                        out_dtype: torch.dtype) -> torch.Tensor:
    """``y * silu(gate)`` first, then the RMS norm of each run of ``group`` values (``group`` 0: whole rows) times
    ``weight`` (one gain per column), in fp32 arithmetic; ``[T, N]`` in ``out_dtype``."""
    z = y.float() * F.silu(gate.float())
    g = z.unflatten(-1, (-1, group)) if group > 0 else z.unsqueeze(-2)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    return (g.flatten(-2) * weight.float()).to(out_dtype)


def joint_norm_cache(x: torch.Tensor, num_heads: int, num_kv_heads: int, dim: int, q_norm: torch.Tensor,
                     k_norm: torch.Tensor, eps: float, positions: torch.Tensor, temp_coef: float, temp_every: int,
                     k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                     slot_mapping: Optional[torch.Tensor]) -> torch.Tensor:
    """What lies between the fused projection ``x[T, >= (H + Hkv) * dim]`` = ``[q | k]`` and the attention of a layer
    whose values are its keys: the RMS norm of q over ALL heads at once with ``q_norm[H * dim]`` (and of k with
    ``k_norm[Hkv * dim]``), q times ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)`` at position ``p``
    (``temp_every`` 0: no such factor), normed k into the key rows ``k_cache[blocks, Hkv, block, dim]`` and k AS
    PROJECTED into the values ``v_cache[blocks, Hkv, block / 8, dim, 8]``.  Returns ``q[T, H, dim]`` in ``x``'s
    dtype."""
    t = x.shape[0]
    qs, ks = num_heads * dim, num_kv_heads * dim
    xf = x[:, :qs + ks].float()
    q, k = xf[:, :qs], xf[:, qs:]
    qn = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()
    kn = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm.float()
    if temp_every > 0:
        p = positions[:t].long()
        qn = qn * (1.0 + temp_coef * torch.log(torch.div(p + 1, temp_every, rounding_mode="floor").float() + 1.0)).unsqueeze(1)
    if k_cache is not None:
        bs = k_cache.shape[2]
        valid = slot_mapping[:t] >= 0
        sm = slot_mapping[:t][valid].long()
        blk, off = sm // bs, sm % bs
        k_cache[blk, :, off, :] = kn[valid].reshape(-1, num_kv_heads, dim).to(k_cache.dtype)
        v_cache[blk, :, off // V_GROUP, :, off % V_GROUP] = k[valid].reshape(-1, num_kv_heads, dim).to(v_cache.dtype)
    return qn.reshape(t, num_heads, dim).to(x.dtype)


def crossed_bias_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                           query_start_loc: torch.Tensor, seq_lens: torch.Tensor, scale: float,
                           bias_scale: Optional[torch.Tensor], bias_rate: Optional[torch.Tensor]) -> torch.Tensor:
    """Causal softmax attention as ``window_bias_attention`` (no window, cap, sink or gate) in which every query
    head's weights are applied to the values of EVERY key / value head: fp32 ``[T, Hq, Hkv, Dv]``, entry
    ``[t, h, c]`` = ``sum_j weight_h(t, j) v_c(j)``."""
    t, hq, d = q.shape
    hkv, bs, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    g = hq // hkv
    out = torch.zeros((t, hq, hkv, dv), dtype=torch.float32, device=q.device)
    qsl, sls = query_start_loc.tolist(), seq_lens.tolist()
    for i, sl in enumerate(sls):
        s, e = qsl[i], qsl[i + 1]
        ql = e - s
        if ql == 0:
            continue
        blocks = block_table[i, :(sl + bs - 1) // bs].long()
        k = k_cache[blocks].permute(1, 0, 2, 3).reshape(hkv, -1, d)[:, :sl].float().repeat_interleave(g, dim=0)
        v = v_cache[blocks].permute(1, 0, 2, 4, 3).reshape(hkv, -1, dv)[:, :sl].float()
        sc = torch.matmul(q[s:e].float().transpose(0, 1), k.transpose(1, 2)) * scale
        qpos = torch.arange(sl - ql, sl, device=q.device).unsqueeze(1)
        kpos = torch.arange(sl, device=q.device).unsqueeze(0)
        if bias_scale is not None:
            dist = (qpos - kpos).clamp(min=0).float()
            sc = sc - bias_scale.float().view(-1, 1, 1) * torch.log1p(bias_rate.float().view(-1, 1, 1) * dist)
        p = torch.softmax(sc.masked_fill(kpos > qpos, float("-inf")), -1)
        out[s:e] = torch.einsum("hqk,ckd->qhcd", p, v)
    return out


def mix_heads(o: torch.Tensor, talk: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """``o[T, H, Hkv, Dv]`` (head ``g``'s weights on value head ``c``) and ``talk[H, H]``: head ``h`` gets
    ``sum_g talk[h, g] * o[t, g, h // (H / Hkv)]``, which is what mixing the heads' softmax weights by ``talk`` and
    applying them to head ``h``'s own values gives.  fp32 arithmetic; ``[T, H * Dv]`` in ``out_dtype``."""
    t, h, c, dv = o.shape
    own = torch.arange(h, device=o.device) // (h // c)
    picked = o.float()[:, :, own, :]                                # [T, g, h, Dv]
    return torch.einsum("hg,tghd->thd", talk.float(), picked).reshape(t, h * dv).to(out_dtype)
