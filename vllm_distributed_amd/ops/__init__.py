"""Op dispatch: hand-written gfx950 HIP kernels on GPU, PyTorch reference on CPU.

``VDAMD_OPS_BACKEND`` = ``auto`` (default: HIP for CUDA tensors, torch for CPU
tensors), ``hip`` (fail if the extension is missing) or ``torch`` (reference
everywhere).  On a GPU box a missing extension is an error, not a silent
fallback: numbers measured on the reference path would be meaningless.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import envs
from . import torch_ref
from .torch_ref import k_cache_shape, v_cache_shape  # noqa: F401  (the paged-cache layouts every backend shares)

_hip = None
_hip_error: Optional[BaseException] = None


def _load_hip():
    global _hip, _hip_error
    if _hip is not None or _hip_error is not None:
        return _hip
    try:
        from . import hip as hip_mod
        hip_mod.load()
        _hip = hip_mod
    except BaseException as e:  # noqa: BLE001
        _hip_error = e
    return _hip


def hip_available() -> bool:
    return _load_hip() is not None


def hip_supports_head_dim(d: int) -> bool:
    return hip_available() and _hip.supports_head_dim(d)


# How often attention ran on the HIP kernels and how often a GPU tensor took the PyTorch reference instead
# (a head size the kernels are not built for).  Workers report it in ``get_stats``; the reference path is
# announced once per head size, loudly: numbers measured on it say nothing about the kernels.
attention_calls = {"hip": 0, "reference_on_gpu": 0}
_announced_fallbacks = set()


def _note_attention(q, on_hip: bool) -> None:
    if on_hip:
        attention_calls["hip"] += 1
        return
    if not q.is_cuda:
        return
    attention_calls["reference_on_gpu"] += 1
    d = int(q.shape[-1])
    if d not in _announced_fallbacks:
        _announced_fallbacks.add(d)
        from ..logger import init_logger
        init_logger(__name__).warning(
            "attention with head size %d runs on the PyTorch REFERENCE path on the GPU (the HIP kernels are built for "
            "%s): correct, but slow and not hipGraph-friendly", d, sorted(_hip.HEAD_DIMS) if _hip is not None else "?")


def _use_hip(t: torch.Tensor) -> bool:
    if not t.is_cuda:
        return False
    backend = envs.VDAMD_OPS_BACKEND
    if backend == "torch":
        return False
    if _load_hip() is None:
        raise RuntimeError(
            "HIP kernel library is not available on a GPU tensor path "
            f"({_hip_error!r}); build it with `python -m vllm_distributed_amd.build` "
            "or set VDAMD_OPS_BACKEND=torch to use the slow reference ops")
    return True


def rms_norm(x, weight, eps):
    if _use_hip(x):
        return _hip.rms_norm(x, weight, eps)
    return torch_ref.rms_norm(x, weight, eps)


def fused_add_rms_norm(x, residual, weight, eps) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns ``(normed, new_residual)``; the HIP path updates both in place."""
    if _use_hip(x):
        return _hip.fused_add_rms_norm(x, residual, weight, eps)
    return torch_ref.fused_add_rms_norm(x, residual, weight, eps)


def reduce_add_rms_norm(partial, residual, weight, eps) -> Tuple[torch.Tensor, torch.Tensor]:
    """``fused_add_rms_norm`` whose first operand arrives as fp32 K-split slabs ``[ks, T, H]``."""
    if _use_hip(residual):
        return _hip.reduce_add_rms_norm(partial, residual, weight, eps)
    return torch_ref.fused_add_rms_norm(partial.sum(0).to(residual.dtype), residual, weight, eps)


def linear_partials(x, weight):
    """``x @ weight^T`` left as the fp32 K-split slabs ``[ks, M, N]`` of the short-batch kernels, for a
    consumer that reduces them itself (the add + RMSNorm that follows a row-parallel projection); None
    where the shape runs unsplit or on another kernel."""
    if not (x.is_cuda and x.dim() == 2 and 0 < x.shape[0] <= 256 and envs.VDAMD_SKINNY_GEMM
            and envs.VDAMD_FUSED_REDUCE_NORM and _use_hip(x)):
        return None
    m, n, k = x.shape[0], weight.shape[0], weight.shape[1]
    if _hip.mid_profitable(m, n, k) and _hip.mid_supported(x, weight):
        return _hip.mid_gemm(x, weight, partials=True)
    if m <= 128 and _hip.skinny_profitable(m, n, k) and _hip.skinny_supported(x, weight):
        return _hip.skinny_gemm_partials(x, weight)
    return None


def w4a16_partials(x, qw, sz):
    """The fused 4-bit GEMM left as its fp32 K-split slabs (None: unsplit shape or a batch it does not take)."""
    if not (x.dim() == 2 and _use_hip(x) and x.dtype in (torch.bfloat16, torch.float16)
            and 0 < x.shape[0] <= _hip.W4_MAX_FUSED_M and envs.VDAMD_FUSED_REDUCE_NORM):
        return None
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    return _hip.w4a16_gemm(x, qw, sz, partials=True)


def layer_norm(x, weight, bias, eps):
    if _use_hip(x):
        return _hip.layer_norm(x, weight, bias, eps)
    return torch_ref.layer_norm(x, weight, bias, eps)


def silu_and_mul(x):
    if _use_hip(x):
        return _hip.silu_and_mul(x)
    return torch_ref.silu_and_mul(x)


def rotary_embedding(positions, q, k, cos_sin_cache, head_dim):
    # the HIP kernel rotates whole heads; a partial rotation (GPT-NeoX's rotary_pct) takes the reference ops
    if _use_hip(q) and cos_sin_cache.shape[-1] == head_dim:
        return _hip.rotary_embedding(positions, q, k, cos_sin_cache, head_dim)
    return torch_ref.rotary_embedding(positions, q, k, cos_sin_cache, head_dim)


def reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, kv_scales=None):
    """``kv_scales = (k_scale[Hkv], v_scale[Hkv])`` fp32: only read for an e4m3 cache."""
    if _use_hip(k):
        return _hip.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, kv_scales)
    return torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping, kv_scales)


def rope_and_cache(positions, qkv, cos_sin_cache, k_cache, v_cache, slot_mapping,
                   num_heads, num_kv_heads, head_dim, q_norm_weight=None, k_norm_weight=None, norm_eps=0.0,
                   kv_scales=None):
    if _use_hip(qkv):
        return _hip.rope_and_cache(positions, qkv, cos_sin_cache, k_cache, v_cache, slot_mapping,
                                   num_heads, num_kv_heads, head_dim, q_norm_weight, k_norm_weight, norm_eps,
                                   kv_scales)
    return torch_ref.rope_and_cache(positions, qkv, cos_sin_cache, k_cache, v_cache, slot_mapping,
                                    num_heads, num_kv_heads, head_dim, q_norm_weight, k_norm_weight, norm_eps,
                                    kv_scales)


def rope_cache_fused_ok(head_dim: int) -> bool:
    """Whether the HIP rotary + cache kernel takes this head size (per-head norm included)."""
    lanes = head_dim // 16
    return head_dim % 16 == 0 and lanes & (lanes - 1) == 0 and lanes <= 64 and hip_available()


def rope_and_cache_partials(positions, slabs, dtype, cos_sin_cache, k_cache, v_cache, slot_mapping,
                            num_heads, num_kv_heads, head_dim, q_norm_weight=None, k_norm_weight=None, norm_eps=0.0,
                            kv_scales=None):
    """``rope_and_cache`` on a projection left as K-split slabs (``linear_partials`` / ``w4a16_partials``;
    HIP only): returns the rotated ``q``."""
    return _hip.rope_and_cache_partials(positions, slabs, dtype, cos_sin_cache, k_cache, v_cache, slot_mapping,
                                        num_heads, num_kv_heads, head_dim, q_norm_weight, k_norm_weight, norm_eps,
                                        kv_scales)


def paged_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, scale,
                    max_query_len: int = 0, max_seq_len: int = 0, out=None, kv_scales=None, window: int = 0,
                    softcap: float = 0.0, sinks=None, alibi_slopes=None):
    on_hip = _use_hip(q) and _hip.supports_head_dim(q.shape[-1])
    _note_attention(q, on_hip)
    if on_hip:
        return _hip.paged_attention_prefill(q, k_cache, v_cache, block_table, query_start_loc,
                                            seq_lens, scale, max_query_len, max_seq_len, out, kv_scales, window,
                                            softcap, sinks, alibi_slopes)
    res = torch_ref.paged_attention(q, k_cache, v_cache, block_table, query_start_loc,
                                    seq_lens, scale, kv_scales, window, softcap, sinks, alibi_slopes)
    if out is not None:
        out.copy_(res)
        return out
    return res


def paged_attention_decode(q, k_cache, v_cache, block_table, seq_lens, scale,
                           max_seq_len: int = 0, out=None, workspace=None, kv_scales=None, window: int = 0,
                           softcap: float = 0.0, sinks=None, alibi_slopes=None):
    on_hip = _use_hip(q) and _hip.supports_head_dim(q.shape[-1])
    _note_attention(q, on_hip)
    if on_hip:
        return _hip.paged_attention_decode(q, k_cache, v_cache, block_table, seq_lens, scale,
                                           max_seq_len, out, workspace, kv_scales=kv_scales, window=window,
                                           softcap=softcap, sinks=sinks, alibi_slopes=alibi_slopes)
    res = torch_ref.paged_attention_decode(q, k_cache, v_cache, block_table, seq_lens, scale, kv_scales, window,
                                           softcap, sinks, alibi_slopes)
    if out is not None:
        out.copy_(res)
        return out
    return res


def sample(logits, temperature, top_k, top_p, min_p, uniform):
    if _use_hip(logits):
        return _hip.sample(logits, temperature, top_k, top_p, min_p, uniform)
    return torch_ref.sample(logits, temperature, top_k, top_p, min_p, uniform)


def argmax(logits):
    if _use_hip(logits):
        return _hip.argmax(logits)
    return logits.argmax(-1)


def embedding(ids, weight, vocab_start=0, masked=False, out=None):
    if _use_hip(weight):
        return _hip.embedding(ids, weight, vocab_start, out)
    res = torch_ref.embedding(ids, weight, vocab_start, masked)
    if out is not None:
        out.copy_(res)
        return out
    return res


def linear(x, weight, bias=None, out=None):
    """``x @ weight^T (+ bias)``: the library GEMM, except for short batches on
    long-reduction shapes where the weight-streaming HIP kernel is faster.
    ``out`` (2-D ``x`` only): write the result there (e.g. straight into the
    buffer the following all-reduce reads)."""
    if x.is_cuda and x.dim() == 2 and x.shape[0] <= 256 and envs.VDAMD_SKINNY_GEMM and _use_hip(x):
        m, n, k = x.shape[0], weight.shape[0], weight.shape[1]
        if (envs.VDAMD_STREAM_GEMM and _hip.stream_profitable(m, n, k) and _hip.stream_supported(x, weight)
                and (out is None or out.stride(0) == n)):
            y = _hip.stream_gemm(x, weight, out=out)
            return y if bias is None else y.add_(bias)
        if _hip.mid_profitable(m, n, k) and _hip.mid_supported(x, weight):
            y = _hip.mid_gemm(x, weight, out=out)
            return y if bias is None else y.add_(bias)
        if m <= 128 and _hip.skinny_profitable(m, n, k) and _hip.skinny_supported(x, weight):
            y = _hip.skinny_gemm(x, weight, out=out)
            return y if bias is None else y.add_(bias)
    if (x.is_cuda and x.dim() == 2 and envs.VDAMD_BIG_GEMM and _use_hip(x) and x.shape[0] >= _hip.BIG_MIN_M
            and _hip.big_profitable(x.shape[0], weight.shape[0], weight.shape[1])
            and _hip.big_supported(x, weight) and _big_out_ok(out, x.shape[0])):
        y = _hip.big_gemm(x, weight, out=out)
        return y if bias is None else y.add_(bias)
    if out is not None and x.dim() == 2:
        if bias is None:
            return torch.mm(x, weight.t(), out=out)
        return torch.addmm(bias, x, weight.t(), out=out)
    return torch.nn.functional.linear(x, weight, bias)


def linear_f32(x, weight):
    """``x @ weight^T`` with the fp32 accumulators kept as the result (logits that are post-processed in fp32)."""
    if x.dtype == torch.float32:
        return torch.nn.functional.linear(x, weight)
    if x.is_cuda and x.dim() == 2:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    return torch.nn.functional.linear(x.float(), weight.float())


_GELU_KINDS = {"gelu": "none", "gelu_new": "tanh", "gelu_pytorch_tanh": "tanh", "gelu_fast": "tanh",
               "gelu_tanh": "tanh"}


def activation(x, kind: str):
    """Element-wise activation by its Hugging Face name."""
    if kind in ("silu", "swish"):
        return torch.nn.functional.silu(x)
    if kind == "relu":
        return torch.relu(x)
    if kind == "relu2":
        return torch.relu(x).square_()
    if kind in _GELU_KINDS:
        return torch.nn.functional.gelu(x, approximate=_GELU_KINDS[kind])
    raise ValueError(f"unsupported activation {kind!r}")


def act_and_mul(x, kind: str):
    """``act(x[..., :F]) * x[..., F:]`` for a gated MLP with an activation other than SiLU (GeGLU)."""
    if kind in ("silu", "swish"):
        return silu_and_mul(x)
    f = x.shape[-1] // 2
    return activation(x[..., :f], kind) * x[..., f:]


def _big_out_ok(out, m):
    return out is None or (out.stride(1) == 1 and out.stride(0) % 8 == 0 and out.data_ptr() % 16 == 0
                           and m * out.stride(0) * 2 < (1 << 32) - 64)


def linear_split(x, weight, split: int):
    """``x @ weight^T`` as two GEMMs over ``weight[:split]`` and ``weight[split:]`` writing one buffer,
    when the first part alone fills the chip in whole rounds of the large-batch kernel's tiles while the
    whole matrix would not (a 70B qkv projection at 2048 rows: 8192 q columns = 256 tiles = one round,
    10240 = 1.25 rounds; 249 us against 276 us for the library on the whole matrix); None otherwise."""
    if not (x.is_cuda and x.dim() == 2 and envs.VDAMD_BIG_GEMM and _use_hip(x) and x.shape[0] >= _hip.BIG_MIN_M):
        return None
    m, n, k = x.shape[0], weight.shape[0], weight.shape[1]
    if (not 0 < split < n or split % 8 or _hip.big_profitable(m, n, k) or not _hip.big_profitable(m, split, k)
            or not _hip.big_supported(x, weight[:split])):
        return None
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    _hip.big_gemm(x, weight[:split], out=out[:, :split])
    torch.mm(x, weight[split:].t(), out=out[:, split:])
    return out


def linear_add(x, weight, residual) -> bool:
    """``residual += x @ weight^T`` inside the large-batch GEMM (its epilogue reads and rewrites the
    residual tile it has just computed); False when that kernel does not take the shape."""
    if (x.is_cuda and x.dim() == 2 and envs.VDAMD_BIG_GEMM and _use_hip(x) and x.shape[0] >= _hip.BIG_MIN_M
            and _hip.big_profitable(x.shape[0], weight.shape[0], weight.shape[1])
            and _hip.big_supported(x, weight) and residual.shape == (x.shape[0], weight.shape[0])
            and residual.dtype == x.dtype and _big_out_ok(residual, x.shape[0])):
        _hip.big_gemm(x, weight, out=residual, residual=residual)
        return True
    return False


def gate_up_silu(x, weight):
    """``silu(x @ Wg^T) * (x @ Wu^T)`` for ``weight = [Wg ; Wu]`` in one kernel (the large-batch GEMM
    forms the activation in its epilogue: the ``[M, 2F]`` intermediate is never written), or ``None``
    when that kernel does not take the shape - the caller then runs the two-step path.  A handful of rows
    take the barrier-free weight-streaming kernel, which has the same epilogue."""
    if (x.is_cuda and x.dim() == 2 and envs.VDAMD_STREAM_GEMM and envs.VDAMD_SKINNY_GEMM and _use_hip(x)
            and _hip.stream_profitable(x.shape[0], weight.shape[0], weight.shape[1])
            and _hip.stream_supported(x, weight) and weight.shape[0] % 64 == 0):
        return _hip.stream_gemm(x, weight, silu_mul=True)
    if (x.is_cuda and x.dim() == 2 and envs.VDAMD_BIG_GEMM and _use_hip(x) and x.shape[0] >= _hip.BIG_MIN_M_SILU
            and _hip.big_profitable(x.shape[0], weight.shape[0], weight.shape[1], True)
            and _hip.big_supported(x, weight, True)):
        return _hip.big_gemm(x, weight, silu_mul=True)
    return None


def silu_mul_linear(gate_up, weight, out=None):
    """``(silu(gate) * up) @ weight^T`` for ``gate_up = [gate | up]``: one kernel when the
    weight-streaming GEMM takes the shape (it forms the activation while staging its operand),
    otherwise the activation kernel followed by ``linear``."""
    if (gate_up.is_cuda and gate_up.dim() == 2 and gate_up.shape[0] <= 128 and envs.VDAMD_SKINNY_GEMM
            and envs.VDAMD_FUSE_SILU_GEMM and _use_hip(gate_up)):
        m, n, k = gate_up.shape[0], weight.shape[0], weight.shape[1]
        if (gate_up.shape[1] == 2 * k and not _hip.mid_profitable(m, n, k) and _hip.skinny_profitable(m, n, k)
                and _hip.skinny_supported(gate_up[:, :k], weight)):
            return _hip.skinny_gemm(gate_up, weight, out=out, silu_mul=True)
    return linear(silu_and_mul(gate_up), weight, None, out)


FP8_MAX = 448.0        # largest finite OCP e4m3 value


def fp8_quantize_weight(w):
    """Per-output-channel symmetric quantisation of ``w [N, K]`` to e4m3:
    ``(wq float8_e4m3fn, scale [N] fp32)`` with ``w ~ wq * scale[:, None]``."""
    wf = w.to(torch.float32)
    scale = wf.abs().amax(dim=1).clamp_min(1e-12) / FP8_MAX
    wq = (wf / scale.unsqueeze(1)).clamp_(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return wq, scale


def fp8_linear(x, wq, w_scale, bias=None):
    """W8A8 linear: activations quantised per token on the fly (HIP kernel),
    weights per output channel, product on the fp8 matrix cores through
    hipBLASLt (``torch._scaled_mm``, fp32 accumulation, row-wise scaling).
    Off the GPU the same arithmetic is done in fp32 from the dequantised
    operands."""
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    if _use_hip(x2) and x2.dtype in (torch.bfloat16, torch.float16) and x2.shape[0] > 0:
        if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
            x2 = x2.contiguous()
        xq, xs = _hip.dynamic_fp8_quant(x2)
        y = torch._scaled_mm(xq, wq.t(), scale_a=xs, scale_b=w_scale.view(1, -1), bias=bias, out_dtype=x2.dtype)
    else:
        xf = x2.to(torch.float32)
        xs = xf.abs().amax(dim=1, keepdim=True).clamp_min(1e-12) / FP8_MAX
        xq = (xf / xs).clamp_(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
        y = (xq.to(torch.float32) * xs) @ (wq.to(torch.float32) * w_scale.view(-1, 1)).t()
        if bias is not None:
            y = y + bias.to(torch.float32)
        y = y.to(x.dtype)
    return y.view(shape[:-1] + (y.shape[-1],))


_w4_scratch = {}


def _scratch_key(device, dtype):
    d = torch.device(device)
    return (d.index if d.index is not None else torch.cuda.current_device(), dtype)


def w4_reserve_scratch(numel: int, device, dtype) -> None:
    """Size the dequantisation scratch for the largest quantised matrix up
    front: captured hipGraphs keep its address, so it must never be
    reallocated while serving."""
    if torch.device(device).type != "cuda":
        return
    key = _scratch_key(device, dtype)
    buf = _w4_scratch.get(key)
    if buf is None or buf.numel() < numel:
        _w4_scratch[key] = torch.empty(numel, dtype=dtype, device=device)


def w4a16_linear(x, qw, sz, bias=None, dense=None):
    """``y = x . dequant(qw, sz)^T (+ bias)`` for weights packed by
    ``ops.quant.pack_w4``.  Small batches run the fused 4-bit MFMA kernel (the
    weights cross HBM once, as 4-bit); large batches dequantise into a shared
    scratch matrix and use the library GEMM, which is compute-bound there
    (``dense``: a resident dequantised copy to use instead, see
    ``VDAMD_W4_DENSE_SHADOW``)."""
    from . import quant
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    if _use_hip(x2) and x2.dtype in (torch.bfloat16, torch.float16):
        if x2.shape[0] <= _hip.W4_MAX_FUSED_M:
            if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
                x2 = x2.contiguous()
            y = _hip.w4a16_gemm(x2, qw, sz)
        elif dense is not None:
            y = torch.nn.functional.linear(x2, dense)
        else:
            n, k = qw.shape[0] * 16, qw.shape[1] * 128
            key = _scratch_key(x2.device, sz.dtype)
            buf = _w4_scratch.get(key)
            if buf is None or buf.numel() < n * k:
                buf = _w4_scratch[key] = torch.empty(n * k, dtype=sz.dtype, device=x2.device)
            y = torch.nn.functional.linear(x2, _hip.w4_dequant(qw, sz, buf))
    else:
        y = torch.nn.functional.linear(x2, quant.w4_dequant(qw, sz, x2.dtype))
    if bias is not None:
        y = y + bias
    return y.view(shape[:-1] + (y.shape[-1],))


def fp4_linear(x, qw, fs, alpha=None, bias=None, dense=None):
    """``y = x . dequant(qw, fs, alpha)^T (+ bias)`` for NVFP4 weights packed by
    ``ops.quant.pack_fp4`` (weight-only: activations stay bf16/fp16).  Same
    split as ``w4a16_linear``: fused 4-bit kernel for small batches, dequantise
    + library GEMM for large ones."""
    from . import quant
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    if _use_hip(x2) and x2.dtype in (torch.bfloat16, torch.float16):
        if x2.shape[0] <= _hip.W4_MAX_FUSED_M:
            if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
                x2 = x2.contiguous()
            y = _hip.fp4a16_gemm(x2, qw, fs, alpha)
        elif dense is not None:
            y = torch.nn.functional.linear(x2, dense)
        else:
            n, k = qw.shape[0] * 16, qw.shape[1] * 128
            key = _scratch_key(x2.device, x2.dtype)
            buf = _w4_scratch.get(key)
            if buf is None or buf.numel() < n * k:
                buf = _w4_scratch[key] = torch.empty(n * k, dtype=x2.dtype, device=x2.device)
            y = torch.nn.functional.linear(x2, _hip.fp4_dequant(qw, fs, alpha, x2.dtype, buf))
    else:
        y = torch.nn.functional.linear(x2, quant.fp4_dequant(qw, fs, alpha, x2.dtype))
    if bias is not None:
        y = y + bias
    return y.view(shape[:-1] + (y.shape[-1],))


def moe_align(topi, num_experts: int, tile_rows: int, expert_start: int = 0, local_experts: int = -1):
    """Sort the ``T*k`` (token, expert) slots by expert and cut each expert's
    run into row tiles, entirely on the device (no host sync, so a decode
    step with experts stays hipGraph-capturable).

    Returns ``(order, tiles)``: ``order [T*k]`` maps sorted position -> flat
    slot ``t*k + j``; ``tiles [n, 3] int32`` = (local expert, first sorted row,
    rows), ``n = T*k // tile_rows + E`` (an upper bound), rows = 0 for unused
    entries and for experts this rank does not hold."""
    flat = topi.reshape(-1)
    tk = flat.numel()
    order = flat.argsort(stable=True)
    counts = torch.zeros(num_experts, dtype=torch.int64, device=flat.device)
    counts.scatter_add_(0, flat, torch.ones_like(flat))
    ends = counts.cumsum(0)
    tpe = (counts + tile_rows - 1) // tile_rows
    tends = tpe.cumsum(0)
    n = tk // tile_rows + num_experts
    j = torch.arange(n, device=flat.device)
    e = torch.searchsorted(tends, j, right=True).clamp_(max=num_experts - 1)
    within = j - (tends - tpe)[e]
    row0 = (ends - counts)[e] + within * tile_rows
    rows = (counts[e] - within * tile_rows).clamp_(min=0, max=tile_rows)
    rows = torch.where(j < tends[-1], rows, torch.zeros_like(rows))
    if local_experts >= 0:
        local = (e >= expert_start) & (e < expert_start + local_experts)
        rows = torch.where(local, rows, torch.zeros_like(rows))
        e = (e - expert_start).clamp_(min=0, max=max(local_experts - 1, 0))
    tiles = torch.stack([e, row0, rows], dim=1).to(torch.int32).contiguous()
    return order, tiles


def moe_route_fused_ok(logits, num_experts: int, top_k: int) -> bool:
    """Whether the three-kernel HIP routing path (``csrc/moe_route.hip``) covers this router."""
    return (_use_hip(logits) and logits.dim() == 2 and num_experts <= _hip.MOE_MAX_EXPERTS
            and top_k <= _hip.MOE_MAX_TOPK and logits.dtype in (torch.bfloat16, torch.float16, torch.float32))


def moe_topk(logits, k: int, renormalize: bool):
    return _hip.moe_topk(logits, k, renormalize)


def moe_topk_grouped(logits, bias, k: int, n_group: int, topk_group: int, sigmoid: bool, group_top2: bool,
                     renormalize: bool, scale: float):
    return _hip.moe_topk_grouped(logits, bias, k, n_group, topk_group, sigmoid, group_top2, renormalize, scale)


def moe_align_fused(topi, num_experts: int, tile_rows: int, expert_start: int = 0, local_experts: int = -1):
    return _hip.moe_align(topi, num_experts, tile_rows, expert_start, local_experts)


def moe_route_small_ok(logits, x) -> bool:
    """Whether the one-launch routing path takes this (decode-sized) batch (``logits`` None: not computed yet)."""
    return (x.dim() == 2 and 0 < x.shape[0] <= _hip.MOE_SMALL_MAX_TOKENS and x.dtype in (torch.bfloat16, torch.float16)
            and (logits is None or logits.dtype in (x.dtype, torch.float32)) and x.stride(1) == 1
            and x.stride(0) % 8 == 0 and x.shape[1] % 8 == 0 and x.data_ptr() % 16 == 0)


def router_logit_partials(x, weight):
    """Router GEMM for a decode-sized batch with its K-split reduction left to the routing kernel: fp32
    ``[splits, T, E]``, or None when the plain GEMM should run."""
    if not (_use_hip(x) and weight.dtype == x.dtype and moe_route_small_ok(None, x)):
        return None
    return _hip.skinny_gemm_partials(x, weight)


def moe_route_small(logits, x, k: int, renormalize: bool, tile_rows: int, expert_start: int = 0,
                    local_experts: int = -1):
    return _hip.moe_route_small(logits, x, k, renormalize, tile_rows, expert_start, local_experts)


def moe_combine(y, topw, topi, inv, expert_start: int = 0, local_experts: int = -1, bias=None):
    return _hip.moe_combine(y, topw, topi, inv, expert_start, local_experts, bias)


def bias_clamped_glu(h, bias, topi, inv, expert_start: int, local_experts: int, limit: float, alpha: float):
    """gpt-oss expert activation with the per-expert bias, on expert-sorted rows (HIP only)."""
    return _hip.bias_clamped_glu(h, bias, topi, inv, expert_start, local_experts, limit, alpha)


def moe_combine_add_rms_norm(y, topw, topi, inv, expert_start, local_experts, residual, weight, eps):
    """``fused_add_rms_norm(moe_combine(...), residual, weight, eps)`` in one launch (HIP only)."""
    return _hip.moe_combine_add_rms_norm(y, topw, topi, inv, expert_start, local_experts, residual, weight, eps)


def grouped_linear(x, tiles, tile_rows: int, weight=None, qw=None, sz=None, alpha=None, silu_mul: bool = False):
    """Row-grouped ``x @ W[g]^T`` (dense ``weight [G, N, K]``, packed 4-bit
    integer ``qw/sz``, or NVFP4 ``qw`` + int32 ``sz`` + ``alpha [G, N]``) for rows
    sorted by group - see ``moe_align``.  HIP only.  ``silu_mul``: ``x`` is ``[rows, 2K] = [gate | up]``
    and the product is taken with ``silu(gate) * up`` (inside the kernel where ``grouped_silu_fused`` says
    so, through the activation kernel otherwise)."""
    assert _use_hip(x)
    if silu_mul and not grouped_silu_fused(tile_rows, qw, sz):
        x, silu_mul = silu_and_mul(x), False
    if qw is not None:
        if sz.dtype == torch.int32:
            return _hip.grouped_fp4a16_gemm(x, qw, sz, alpha, tiles, tile_rows)
        return _hip.grouped_w4a16_gemm(x, qw, sz, tiles, tile_rows, silu_mul=silu_mul)
    return _hip.grouped_gemm(x, weight, tiles, tile_rows)


def grouped_silu_fused(tile_rows: int, qw, sz) -> bool:
    """Whether the grouped GEMM of these weights forms ``silu(gate) * up`` itself at this tile size
    (integer 4-bit experts, few rows per expert: decode)."""
    return (qw is not None and sz.dtype != torch.int32 and tile_rows <= _hip.W4_GROUPED_SILU_MAX_ROWS
            and envs.VDAMD_MOE_FUSED_SILU)


apply_penalties = torch_ref.apply_penalties
compute_logprobs = torch_ref.compute_logprobs
build_cos_sin_cache = torch_ref.build_cos_sin_cache


# ------------------------------------------------ multi-head latent attention over a latent cache (DeepSeek)
def mla_kernel_ok(dk: int, dv: int, dtype: torch.dtype) -> bool:
    """Whether the HIP latent-attention kernel is built for this key / value width."""
    return hip_available() and _hip.mla_supported(dk, dv, dtype)


def mla_cache_write(latent, k_cache, v_cache, slot_mapping):
    if _use_hip(latent) and latent.dtype in (torch.bfloat16, torch.float16):
        return _hip.mla_cache_write(latent, k_cache, v_cache, slot_mapping)      # (the cache may be e4m3)
    return torch_ref.mla_cache_write(latent, k_cache, v_cache, slot_mapping)


def mla_attention(q, k_cache, v_cache, block_table, token_seq, seq_lens, scale, max_seq_len, out=None,
                  precise: bool = False, window: int = 0, sinks=None, gate=None):
    """``precise``: softmax weights with fp32 precision in the weighted sum (models that define them in 32-bit).
    ``window`` / ``sinks`` / ``gate``: a sliding window, a sink per head in the denominator, a sigmoid gate per
    (token, head) on the output (the matrix-core kernels only)."""
    on_hip = _use_hip(q) and _hip.mla_supported(q.shape[2], v_cache.shape[2] * v_cache.shape[4], q.dtype)
    _note_attention(q, on_hip)
    if on_hip:
        return _hip.mla_attention(q, k_cache, v_cache, block_table, token_seq, seq_lens, scale, max_seq_len, out,
                                  precise=precise, window=window, sinks=sinks, gate=gate)
    if window or sinks is not None or gate is not None:
        raise NotImplementedError("window, sinks and gate exist in the matrix-core latent kernels only: layers that "
                                  "use them elsewhere go through latent_row_attention")
    return torch_ref.mla_attention(q, k_cache, v_cache, block_table, token_seq, seq_lens, scale, max_seq_len, out)


def mla_prep_ok(x: torch.Tensor) -> bool:
    """Whether the one-launch query assembly + latent cache write (HIP) takes this tensor."""
    return _use_hip(x) and x.dtype in (torch.bfloat16, torch.float16)


def mla_prep(q, nope, q_lat, latent, norm_weight, eps, cos_sin, positions, k_cache, v_cache, slot_mapping):
    return _hip.mla_prep(q, nope, q_lat, latent, norm_weight, eps, cos_sin, positions, k_cache, v_cache, slot_mapping)


# ------------------------------------------------ single-gain norms, PolyNorm, convolved q/k/v, windowed attention
def embed_positions(ids, positions, embed, pos):
    """``embed[ids] + pos[positions]`` summed in fp32: the residual stream of a model with learned positions."""
    if _use_hip(embed):
        return _hip.embed_positions(ids, positions, embed, pos)
    return embed[ids.long()].float() + pos[positions.long()].float()


def scalar_rms_norm(x, gain, eps: float, out_dtype):
    """RMS norm with one gain for the whole row (fp32 arithmetic), result in ``out_dtype``."""
    if _use_hip(x):
        return _hip.scalar_rms_norm(x, gain, eps, out_dtype)
    return torch_ref.scalar_rms_norm(x, gain, eps, out_dtype)


def scalar_norm_residual(y, post_gain, residual, next_gain, eps: float, out_dtype):
    """``residual += norm(y) * post_gain`` on the fp32 residual stream, and (with ``next_gain``) the normed input of
    the next sublayer in ``out_dtype``: one launch."""
    if _use_hip(y):
        return _hip.scalar_norm_residual(y, post_gain, residual, next_gain, eps, out_dtype)
    return torch_ref.scalar_norm_residual(y, post_gain, residual, next_gain, eps, out_dtype)


def poly_norm(z, coef, eps: float):
    if _use_hip(z):
        return _hip.poly_norm(z, coef, eps)
    return torch_ref.poly_norm(z, coef, eps)


def conv_norm_cache(x, conv_weight, state, slots, query_start_loc, seq_lens, token_seq, positions, num_heads: int,
                    num_kv_heads: int, dim: int, vdim: int, q_norm, k_norm, eps: float, v_first, v_lambda,
                    keep_v: bool, k_cache, v_cache, slot_mapping, has_prefill: bool = True, inv_freq=None):
    """``conv_weight`` is tap-major, ``[taps, C]``.  Short convolution (with per-request state) + per-head q / k norm + value mixing + cache write over a fused
    projection; see ``torch_ref.conv_norm_cache``.  ``token_seq`` (None: row ``t`` belongs to sequence ``t``) and
    ``positions`` tell the kernel which sequence and position each row has.  ``q_norm`` / ``k_norm`` None: no head
    norm; ``inv_freq``: q and k heads are rotated (pairs half a rotation width apart) after the convolution."""
    if _use_hip(x):
        return _hip.conv_norm_cache(x, conv_weight, state, slots, query_start_loc, seq_lens, token_seq, positions,
                                    num_heads, num_kv_heads, dim, vdim, q_norm, k_norm, eps, v_first, v_lambda,
                                    keep_v, k_cache, v_cache, slot_mapping, has_prefill, inv_freq)
    return torch_ref.conv_norm_cache(x, conv_weight, state, slots, query_start_loc, seq_lens, num_heads,
                                     num_kv_heads, dim, vdim, q_norm, k_norm, eps, v_first, v_lambda, keep_v,
                                     k_cache, v_cache, slot_mapping, inv_freq, positions)


def window_bias_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, token_seq, positions,
                          scale: float, softcap: float, window: int, keep_first: int, bias_scale, bias_rate, sinks,
                          gate, max_query_len: int = 0, out=None, chunk: int = 0):
    """Attention over row caches with a window that keeps the first keys (or, ``chunk > 0``, a mask of blocks of
    ``chunk`` positions), a logarithmic distance bias, a sink in the denominator and an output gate; see
    ``torch_ref.window_bias_attention``."""
    if _use_hip(q):
        attention_calls["hip"] += 1
        return _hip.window_bias_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, token_seq,
                                          positions, scale, softcap, window, keep_first, bias_scale, bias_rate, sinks,
                                          gate, max_query_len, out, chunk)
    res = torch_ref.window_bias_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, scale,
                                          softcap, window, keep_first, bias_scale, bias_rate, sinks, gate, chunk)
    if out is not None:
        out.copy_(res)
        return out
    return res


# ------------------------------------------------ fp32 residual stream with layer norms, decayed linear attention,
# ------------------------------------------------ gated norm, clamped GLU, latent attention over one row cache
def embed_scaled(ids, weight, scale: float):
    """``weight[ids] * scale`` as the fp32 residual stream."""
    if _use_hip(weight):
        return _hip.embed_scaled(ids, weight, scale)
    return torch_ref.embed_scaled(ids, weight, scale)


def layer_norm_to(x, weight, bias, eps: float, out_dtype):
    """Layer norm in fp32 arithmetic of rows of any float type, result in ``out_dtype``."""
    if _use_hip(x):
        return _hip.layer_norm_to(x, weight, bias, eps, out_dtype)
    return torch_ref.layer_norm_to(x, weight, bias, eps, out_dtype)


def add_layer_norm(y, residual, weight, bias, eps: float, out_dtype):
    """``residual += y`` on the fp32 residual stream and the layer norm of the sum in ``out_dtype``: one launch."""
    if _use_hip(y):
        return _hip.add_layer_norm(y, residual, weight, bias, eps, out_dtype)
    return torch_ref.add_layer_norm(y, residual, weight, bias, eps, out_dtype)


def decay_linear_attention(x, num_heads: int, dim: int, vdim: int, decay, state, slots, query_start_loc, seq_lens,
                           silu: bool = True, max_query_len: int = 0):
    """Linear attention with a per-head decay and a per-request fp32 state; see
    ``torch_ref.decay_linear_attention``.  ``max_query_len`` (0: unknown) only helps the kernel choose its launch."""
    if _use_hip(x):
        return _hip.decay_linear_attention(x, num_heads, dim, vdim, decay, state, slots, query_start_loc, seq_lens,
                                           silu, max_query_len)
    return torch_ref.decay_linear_attention(x, num_heads, dim, vdim, decay, state, slots, query_start_loc, seq_lens, silu)


def gated_rms_norm(o, weight, gate, eps: float, out_dtype, group: int = 0, scale: float = 1.0, out=None):
    """RMS norm of fp32 rows (whole rows, or runs of ``group`` values sharing ``weight[group]``) times
    ``sigmoid(gate) * scale``; ``out``: a view with strided rows that receives the result."""
    if _use_hip(o):
        return _hip.gated_rms_norm(o, weight, gate, eps, out_dtype, group, scale, out)
    return torch_ref.gated_rms_norm(o, weight, gate, eps, out_dtype, group, scale, out)


def clamped_glu(h, limit: float, alpha: float):
    if _use_hip(h):
        return _hip.clamped_glu(h, limit, alpha)
    return torch_ref.clamped_glu(h, limit, alpha)


def relu_squared(x):
    if _use_hip(x):
        return _hip.relu_squared(x)
    return torch.relu(x).square_()


def latent_prep(q, nope: int, q_lat, latent, norm_weight, eps: float, inv_freq, rot_scale: float, positions, cache,
                slot_mapping, fragments=None, interleaved: bool = False):
    if _use_hip(q):
        return _hip.latent_prep(q, nope, q_lat, latent, norm_weight, eps, inv_freq, rot_scale, positions, cache,
                                slot_mapping, fragments, interleaved)
    return torch_ref.latent_prep(q, nope, q_lat, latent, norm_weight, eps, inv_freq, rot_scale, positions, cache,
                                 slot_mapping, fragments, interleaved)


def latent_row_attention(q, cache, block_table, token_seq, seq_lens, scale: float, rank: int, max_seq_len: int = 0,
                         window: int = 0, sinks=None, gate=None):
    if _use_hip(q):
        attention_calls["hip"] += 1
        return _hip.latent_row_attention(q, cache, block_table, token_seq, seq_lens, scale, rank, max_seq_len,
                                         window, sinks, gate)
    return torch_ref.latent_row_attention(q, cache, block_table, token_seq, seq_lens, scale, rank, window, sinks, gate)


def expert_epilogue(routed, x, topw, topi, real_experts: int, shared, gate):
    """What follows the routed experts of a block with identity experts and a gated shared expert, in one pass; see
    ``torch_ref.expert_epilogue``."""
    if _use_hip(routed) and (topi is None or topi.dtype == torch.int32):
        return _hip.expert_epilogue(routed, x, topw, topi, real_experts, shared, gate)
    return torch_ref.expert_epilogue(routed, x, topw, topi, real_experts, shared, gate)


# ------------------------------------------------ fp32 residual stream with offset RMS norms, side inputs per token,
# ------------------------------------------------ convolutions with activation, the gated delta rule
def rms_norm_to(x, weight, eps: float, out_dtype, offset: float = 0.0):
    """RMS norm in fp32 arithmetic of rows of any float type with fp32 gains ``offset + weight``; see
    ``torch_ref.rms_norm_to``."""
    if _use_hip(x):
        return _hip.rms_norm_to(x, weight, eps, out_dtype, offset)
    return torch_ref.rms_norm_to(x, weight, eps, out_dtype, offset)


def add_rms_norm_to(residual, a, b, weight, eps: float, out_dtype, offset: float = 0.0, normed: bool = True):
    """``residual += a + b`` on the fp32 residual stream and the RMS norm of the sum (or the sum itself) in
    ``out_dtype``: one launch."""
    if _use_hip(residual):
        return _hip.add_rms_norm_to(residual, a, b, weight, eps, out_dtype, offset, normed)
    return torch_ref.add_rms_norm_to(residual, a, b, weight, eps, out_dtype, offset, normed)


def norm_add_norm(y, post_weight, residual, next_weight, eps: float, out_dtype, next_offset: float = 0.0,
                  next_normed: bool = True):
    """``residual += rms_norm(y) * post_weight`` on the fp32 residual stream and the RMS norm of the sum (or the sum
    itself) in ``out_dtype``: one launch."""
    if _use_hip(y):
        return _hip.norm_add_norm(y, post_weight, residual, next_weight, eps, out_dtype, next_offset, next_normed)
    return torch_ref.norm_add_norm(y, post_weight, residual, next_weight, eps, out_dtype, next_offset, next_normed)


def gelu_mul_rows(g, table, ids, col: int):
    if _use_hip(g):
        return _hip.gelu_mul_rows(g, table, ids, col)
    return torch_ref.gelu_mul_rows(g, table, ids, col)


def sigmoid_mul(o, gate, scale: float = 1.0, out=None):
    if _use_hip(o):
        return _hip.sigmoid_mul(o, gate, scale, out)
    return torch_ref.sigmoid_mul(o, gate, scale, out)


def gelu(x, tanh: bool):
    """GELU (the tanh form or the exact one) in fp32 arithmetic, in ``x``'s dtype."""
    if _use_hip(x):
        return _hip.gelu(x, tanh)
    return torch.nn.functional.gelu(x.float(), approximate="tanh" if tanh else "none").to(x.dtype)


def short_conv_act(x, channels: int, conv_weight, state, slots, query_start_loc, seq_lens, token_seq, positions,
                   silu: bool, has_prefill: bool = True, bias=None, residual: bool = False):
    """Causal convolution over time (tap-major ``conv_weight[taps, channels]``, per-request state) of the first
    ``channels`` columns of a fused projection, plus ``bias``, through SiLU when asked, plus the input itself with
    ``residual``; see ``torch_ref.short_conv_act``."""
    if _use_hip(x):
        return _hip.short_conv_act(x, channels, conv_weight, state, slots, query_start_loc, seq_lens, token_seq,
                                   positions, silu, has_prefill, bias, residual)
    return torch_ref.short_conv_act(x, channels, conv_weight, state, slots, query_start_loc, seq_lens, silu, bias,
                                    residual)


def gated_delta_rule(x, num_heads: int, num_qk_heads: int, dim: int, vdim: int, beta, dt, dt_bias, a_log, state,
                     slots, query_start_loc, seq_lens, norm_eps: float = 1e-6, max_query_len: int = 0):
    """The gated delta rule with a decay per head and key channel and a per-request fp32 state; see
    ``torch_ref.gated_delta_rule``."""
    if _use_hip(x):
        return _hip.gated_delta_rule(x, num_heads, num_qk_heads, dim, vdim, beta, dt, dt_bias, a_log, state, slots,
                                     query_start_loc, seq_lens, norm_eps, max_query_len)
    return torch_ref.gated_delta_rule(x, num_heads, num_qk_heads, dim, vdim, beta, dt, dt_bias, a_log, state, slots,
                                      query_start_loc, seq_lens, norm_eps)


# ------------------------------------------------ selective state-space scan, gate in front of a grouped norm,
# ------------------------------------------------ q / k normed over all heads with values = keys, crossed value
# ------------------------------------------------ heads and mixed head weights
def selective_scan(x, dt, num_heads: int, groups: int, vdim: int, n_state: int, a_log, dt_bias, d_skip, state, slots,
                   query_start_loc, seq_lens, max_query_len: int = 0):
    """A state-space recurrence with a data-dependent decay per head and a per-request fp32 state; see
    ``torch_ref.selective_scan``."""
    if _use_hip(x):
        return _hip.selective_scan(x, dt, num_heads, groups, vdim, n_state, a_log, dt_bias, d_skip, state, slots,
                                   query_start_loc, seq_lens, max_query_len)
    return torch_ref.selective_scan(x, dt, num_heads, groups, vdim, n_state, a_log, dt_bias, d_skip, state, slots,
                                    query_start_loc, seq_lens)


def act_gate_group_norm(y, gate, weight, eps: float, group: int, out_dtype):
    """``rms_norm_by_groups(y * silu(gate)) * weight``; see ``torch_ref.act_gate_group_norm``."""
    if _use_hip(y):
        return _hip.act_gate_group_norm(y, gate, weight, eps, group, out_dtype)
    return torch_ref.act_gate_group_norm(y, gate, weight, eps, group, out_dtype)


def joint_norm_cache(x, num_heads: int, num_kv_heads: int, dim: int, q_norm, k_norm, eps: float, positions,
                     temp_coef: float, temp_every: int, k_cache, v_cache, slot_mapping):
    """q and k normed over all their heads at once, the query's position factor, normed k into the key rows and the
    projected k into the values; see ``torch_ref.joint_norm_cache``."""
    if _use_hip(x):
        return _hip.joint_norm_cache(x, num_heads, num_kv_heads, dim, q_norm, k_norm, eps, positions, temp_coef,
                                     temp_every, k_cache, v_cache, slot_mapping)
    return torch_ref.joint_norm_cache(x, num_heads, num_kv_heads, dim, q_norm, k_norm, eps, positions, temp_coef,
                                      temp_every, k_cache, v_cache, slot_mapping)


def crossed_bias_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, token_seq, positions,
                           scale: float, bias_scale, bias_rate, max_query_len: int = 0, out=None):
    """Every query head's softmax weights on every value head, fp32 ``[T, Hq, Hkv, Dv]``; see
    ``torch_ref.crossed_bias_attention``."""
    if _use_hip(q):
        attention_calls["hip"] += 1
        return _hip.window_bias_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, token_seq,
                                          positions, scale, 0.0, 0, 0, bias_scale, bias_rate, None, None,
                                          max_query_len, out, 0, crossed=True)
    res = torch_ref.crossed_bias_attention(q, k_cache, v_cache, block_table, query_start_loc, seq_lens, scale,
                                           bias_scale, bias_rate)
    if out is not None:
        out.copy_(res)
        return out
    return res


def mix_heads(o, talk, out_dtype):
    """Heads mixed by ``talk[H, H]`` over crossed attention outputs; see ``torch_ref.mix_heads``."""
    if _use_hip(o):
        return _hip.mix_heads(o, talk, out_dtype)
    return torch_ref.mix_heads(o, talk, out_dtype)
