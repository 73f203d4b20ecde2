"""HIP kernels of ``csrc/state_space.hip`` (state-space scan, gate in front of a grouped norm, q / k normed over all
heads with the projected keys as values, mixed head weights) and what ``csrc/seq_mix.hip`` gained beside them (a bias
and the input itself added by the convolution, every query head's weights on every value head), against the plain
PyTorch fp32 form of the same op (``ops/torch_ref.py``)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from vllm_distributed_amd.ops import torch_ref  # noqa: E402


def _hip():
    from vllm_distributed_amd.ops import hip
    hip.load()
    return hip


def _close(a, b, dtype, scale=1.0):
    tol = 3e-5 if dtype == torch.float32 else 1.2e-2
    err = (a.float() - b.float()).abs().max().item()
    assert err <= tol * scale, err


def _i32(*v):
    return torch.tensor(list(v), dtype=torch.int32, device="cuda")


def _batch(lens, ctx):
    """Sequences that bring ``lens[i]`` rows as the last positions of ``ctx[i] + lens[i]`` tokens."""
    qsl = [0]
    for n in lens:
        qsl.append(qsl[-1] + n)
    pos, seq = [], []
    for i, (n, c) in enumerate(zip(lens, ctx)):
        pos += list(range(c, c + n))
        seq += [i] * n
    return _i32(*qsl), _i32(*[c + n for n, c in zip(lens, ctx)]), _i32(*pos), _i32(*seq)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("c,taps", [(24, 4), (200, 3), (70, 1), (512, 2)])
def test_conv_bias_and_residual(dtype, c, taps):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(c + taps)
    lens, ctx = [1, 5, 1, 9, 2], [3, 0, 0, 7, 1]
    qsl, sls, pos, seq = _batch(lens, ctx)
    t = sum(lens)
    wide = torch.randn(t, c + 16, device="cuda", generator=g).to(dtype)
    w = (torch.randn(taps, c, device="cuda", generator=g) * 0.5).to(dtype)
    bias = torch.randn(c, device="cuda", generator=g)
    slots = _i32(4, 0, 2, 5, 1)
    st0 = torch.randn(7, max(taps - 1, 1), c, device="cuda", generator=g).to(dtype)
    for x in (wide[:, :c], wide[:, 8:8 + c]):
        for silu, b, res in ((True, bias, False), (False, None, True), (True, None, True), (False, bias, False)):
            s1, s2 = st0.clone(), st0.clone()
            got = hip.short_conv_act(x, c, w, s1, slots, qsl, sls, seq, pos, silu, True, b, res)
            want = torch_ref.short_conv_act(x, c, w, s2, slots, qsl, sls, silu, b, res)
            _close(got, want, dtype, 8)
            if taps > 1:
                assert torch.equal(s1, s2)
    # decoded rows only: the kernel moves the state on by itself
    lens, ctx = [1, 1, 1], [5, 0, 2]
    qsl, sls, pos, _ = _batch(lens, ctx)
    x = wide[:3, :c]
    s1, s2 = st0.clone(), st0.clone()
    got = hip.short_conv_act(x, c, w, s1, _i32(6, 1, 3), qsl, sls, None, pos, False, False, bias, True)
    want = torch_ref.short_conv_act(x, c, w, s2, _i32(6, 1, 3), qsl, sls, False, bias, True)
    _close(got, want, dtype, 8)
    if taps > 1:
        assert torch.equal(s1, s2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h,groups,vdim,n", [(4, 2, 32, 16), (6, 3, 24, 40), (2, 1, 80, 64), (8, 8, 64, 128),
                                             (3, 1, 16, 200), (5, 5, 7, 5)])
def test_selective_scan(dtype, h, groups, vdim, n):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(h * 1000 + n)
    inner = h * vdim
    cols = inner + 2 * groups * n
    a_log = torch.rand(h, device="cuda", generator=g) * 2.5 - 2.0
    dt_bias = torch.rand(h, device="cuda", generator=g) * 3 - 3.5
    skip = torch.rand(h, device="cuda", generator=g)
    st0 = torch.randn(6, h, n, vdim, device="cuda", generator=g)
    for lens, ctx, slots in (([1, 37, 1, 12, 2], [9, 0, 0, 30, 4], [3, 0, 5, 1, 2]), ([1, 1, 1], [4, 0, 1], [2, 4, 0]),
                            ([70], [0], [1])):
        qsl, sls, _, _ = _batch(lens, ctx)
        t = sum(lens)
        wide = (torch.randn(t, cols + h + 8, device="cuda", generator=g) * 0.7).to(dtype)
        x, dt = wide[:, :cols], wide[:, cols:cols + h]
        for d in (skip, None):
            s1, s2 = st0.clone(), st0.clone()
            got = hip.selective_scan(x, dt, h, groups, vdim, n, a_log, dt_bias, d, s1, _i32(*slots), qsl, sls, max(lens))
            want = torch_ref.selective_scan(x, dt, h, groups, vdim, n, a_log, dt_bias, d, s2, _i32(*slots), qsl, sls)
            _close(got, want, torch.float32, 40)
            _close(s1, s2, torch.float32, 40)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,group", [(96, 32), (256, 256), (192, 64), (40, 5), (3072, 1536), (4096, 4096), (8192, 8192),
                                     (16400, 16400)])
def test_act_gate_group_norm(dtype, n, group):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(n + group)
    y = torch.randn(9, n, device="cuda", generator=g) * 2
    wide = torch.randn(9, 2 * n + 8, device="cuda", generator=g).to(dtype)
    w = torch.rand(n, device="cuda", generator=g) + 0.5
    for gate in (wide[:, :n], wide[:, n + 8:]):
        _close(hip.act_gate_group_norm(y, gate, w, 1e-5, group, dtype),
               torch_ref.act_gate_group_norm(y, gate, w, 1e-5, group, dtype), dtype, 8)


def _caches(blocks, g, bs, d, dtype, gen):
    k = torch.randn(blocks, g, bs, d, device="cuda", generator=gen).to(dtype)
    v = torch.randn(blocks, g, bs // 8, d, 8, device="cuda", generator=gen).to(dtype)
    return k, v


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h,g,d,every", [(4, 2, 32, 4), (6, 6, 24, 0), (2, 1, 128, 1), (3, 1, 5, 7)])
def test_joint_norm_cache(dtype, h, g, d, every):
    hip = _hip()
    gen = torch.Generator(device="cuda").manual_seed(h * 100 + d)
    t, bs = 11, 16
    wide = (torch.randn(t, (h + g) * d + 8, device="cuda", generator=gen) * 1.5).to(dtype)
    x = wide[:, :(h + g) * d]
    qw = torch.rand(h * d, device="cuda", generator=gen) + 0.5
    kw = torch.rand(g * d, device="cuda", generator=gen) + 0.5
    pos = _i32(0, 1, 2, 3, 4, 5, 30, 31, 32, 7, 63)
    slots = _i32(5, 17, 18, -1, 40, 41, 42, 0, 63, 9, 33)
    k1, v1 = _caches(4, g, bs, d, dtype, gen)
    k2, v2 = k1.clone(), v1.clone()
    got = hip.joint_norm_cache(x, h, g, d, qw, kw, 1e-5, pos, 0.3, every, k1, v1, slots)
    want = torch_ref.joint_norm_cache(x, h, g, d, qw, kw, 1e-5, pos, 0.3, every, k2, v2, slots)
    _close(got, want, dtype, 8)
    _close(k1, k2, dtype, 8)
    assert torch.equal(v1, v2)                      # the values are copies of the projection
    _close(hip.joint_norm_cache(x, h, g, d, qw, kw, 1e-5, pos, 0.3, every, None, None, None), want, dtype, 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h,g,d", [(4, 2, 32), (6, 3, 64), (4, 4, 16), (2, 1, 128), (3, 3, 24), (8, 2, 64), (8, 4, 128),
                                   (16, 8, 32), (10, 2, 32), (5, 5, 64), (36, 1, 32), (12, 4, 64), (12, 6, 32)])
def test_crossed_attention_and_mixing(dtype, h, g, d):
    hip = _hip()
    gen = torch.Generator(device="cuda").manual_seed(h * 100 + d)
    bs, blocks = 16, 24
    k, v = _caches(blocks, g, bs, d, dtype, gen)
    r1 = torch.rand(h, device="cuda", generator=gen)
    r2 = torch.rand(h, device="cuda", generator=gen)
    talk = torch.eye(h, device="cuda") + torch.randn(h, h, device="cuda", generator=gen) * 0.3
    table = torch.randperm(blocks, device="cuda", generator=gen).to(torch.int32).view(4, 6)
    # prompt portions (token rows), then decoded rows
    for lens, ctx in (([19, 1, 40, 2], [0, 77, 30, 5]), ([1, 1, 1], [90, 0, 33])):
        qsl, sls, pos, seq = _batch(lens, ctx)
        t = sum(lens)
        q = (torch.randn(t, h, d, device="cuda", generator=gen) * 1.5).to(dtype)
        decode = max(lens) == 1
        got = hip.window_bias_attention(q, k, v, table[:len(lens)], qsl, sls, None if decode else seq, pos, 0.2, 0.0, 0,
                                        0, r1, r2, None, None, max(lens), None, 0, crossed=True)
        want = torch_ref.crossed_bias_attention(q, k, v, table[:len(lens)], qsl, sls, 0.2, r1, r2)
        assert got.dtype == torch.float32 and got.shape == (t, h, g, d)
        _close(got, want, dtype, 4)
        _close(hip.mix_heads(want, talk, dtype), torch_ref.mix_heads(want, talk, dtype), dtype, 8)
    # an identity mixing matrix gives each head its own key / value head's column back
    own = torch.arange(h, device="cuda") // (h // g)
    plain = want[:, torch.arange(h, device="cuda"), own]
    _close(hip.mix_heads(want, torch.eye(h, device="cuda"), torch.float32), plain.reshape(want.shape[0], -1),
           torch.float32)


@pytest.mark.parametrize("h,g,d", [(8, 4, 64), (16, 8, 32), (4, 4, 128), (12, 4, 32)])
def test_crossed_decode_with_a_workgroup_per_cu_or_more(h, g, d):
    """Enough decoded sequences that the launch gives a workgroup's wave sets four key heads each (bf16, key heads a
    multiple of 4): contexts of every length from one key to several pages, sequences that are no multiple of 8."""
    hip = _hip()
    dtype = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(h + d)
    bs, nseq, per = 16, 300, 9
    k, v = _caches(nseq * per, g, bs, d, dtype, gen)
    r1 = torch.rand(h, device="cuda", generator=gen)
    r2 = torch.rand(h, device="cuda", generator=gen)
    table = torch.randperm(nseq * per, device="cuda", generator=gen).to(torch.int32).view(nseq, per)
    ctx = [(7 * i) % (bs * per - 1) for i in range(nseq)]
    qsl, sls, pos, _ = _batch([1] * nseq, ctx)
    q = (torch.randn(nseq, h, d, device="cuda", generator=gen) * 1.5).to(dtype)
    got = hip.window_bias_attention(q, k, v, table, qsl, sls, None, pos, 0.2, 0.0, 0, 0, r1, r2, None, None, 1, None, 0,
                                    crossed=True)
    want = torch_ref.crossed_bias_attention(q, k, v, table, qsl, sls, 0.2, r1, r2)
    _close(got, want, dtype, 4)
