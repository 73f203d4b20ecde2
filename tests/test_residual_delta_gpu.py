"""HIP kernels of ``csrc/residual_rms.hip`` and ``csrc/delta_rule.hip``, and what ``csrc/seq_mix.hip`` and
``csrc/linear_latent.hip`` gained beside them (convolution with rotation and without head norms, convolution +
activation, chunked masks, windowed latent rows with sink and gate, neighbouring rotation pairs, the per-head gated
norm), against the plain PyTorch fp32 form of the same op (``ops/torch_ref.py``)."""
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h", [22, 192, 1000, 4096])
def test_residual_norms(dtype, h):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(h)
    x = torch.randn(7, h, device="cuda", generator=g) * 3 + 0.5
    w = torch.randn(h, device="cuda", generator=g) * 0.2
    pw = torch.rand(h, device="cuda", generator=g) + 0.3
    _close(hip.rms_norm_to(x, w, 1e-5, dtype, 1.0), torch_ref.rms_norm_to(x, w, 1e-5, dtype, 1.0), dtype, 4)
    wide = torch.randn(7, 3 * h + 8, device="cuda", generator=g).to(dtype)
    a, b, y = wide[:, :h], wide[:, h:2 * h], wide[:, 2 * h + 8:]          # strided views, as fused projections give
    _close(hip.rms_norm_to(a, pw, 1e-5, dtype), torch_ref.rms_norm_to(a, pw, 1e-5, dtype), dtype, 4)
    for second in (b, None):
        for normed in (True, False):
            r1, r2 = x.clone(), x.clone()
            o1 = hip.add_rms_norm_to(r1, a, second, w, 1e-5, dtype, 1.0, normed)
            o2 = torch_ref.add_rms_norm_to(r2, a, second, w, 1e-5, dtype, 1.0, normed)
            _close(r1, r2, torch.float32, 8)
            _close(o1, o2, dtype, 8)
    for normed in (True, False):
        r1, r2 = x.clone(), x.clone()
        o1 = hip.norm_add_norm(y, pw, r1, w, 1e-5, dtype, 1.0, normed)
        o2 = torch_ref.norm_add_norm(y, pw, r2, w, 1e-5, dtype, 1.0, normed)
        _close(r1, r2, torch.float32, 8)
        _close(o1, o2, dtype, 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n", [5, 16, 64, 128, 136])
def test_gates_and_activations(dtype, n):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(n)
    wide = (torch.randn(9, 3 * n, device="cuda", generator=g) * 2).to(dtype)
    o, gate = wide[:, :n], wide[:, 2 * n:]
    dst = torch.zeros(9, 2 * n + 3, device="cuda", dtype=dtype)
    hip.sigmoid_mul(o, gate, 0.6, out=dst[:, n:2 * n])
    _close(dst[:, n:2 * n], torch_ref.sigmoid_mul(o, gate, 0.6), dtype, 4)
    assert float(dst[:, :n].abs().max()) == 0 and float(dst[:, 2 * n:].abs().max()) == 0
    _close(hip.sigmoid_mul(o, gate), torch_ref.sigmoid_mul(o, gate), dtype, 4)
    x = (torch.randn(11, n, device="cuda", generator=g) * 2.5).to(dtype)
    for tanh in (True, False):
        want = torch.nn.functional.gelu(x.float(), approximate="tanh" if tanh else "none")
        _close(hip.gelu(x, tanh), want, dtype, 4)
    table = torch.randn(13, 4 * n, device="cuda", generator=g).to(dtype)
    ids = _i32(3, 0, 12, 3, 7, 1, 1, 9, 5)
    _close(hip.gelu_mul_rows(gate, table, ids, 2 * n), torch_ref.gelu_mul_rows(gate, table, ids, 2 * n), dtype, 8)
    heads = torch.randn(9, 3 * n, device="cuda", generator=g) * 2
    wgt = torch.rand(n, device="cuda", generator=g) + 0.5
    dst = torch.zeros(9, 3 * n + 8, device="cuda", dtype=dtype)
    hip.gated_rms_norm(heads, wgt, wide, 1e-5, dtype, n, 0.5, dst[:, 8:])
    _close(dst[:, 8:], torch_ref.gated_rms_norm(heads, wgt, wide, 1e-5, dtype, n, 0.5), dtype, 4)
    assert float(dst[:, :8].abs().max()) == 0


def _conv_case(dtype, t_sizes, starts, channels, taps, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = sum(t_sizes)
    x = torch.randn(t, channels + 10, device="cuda", generator=g).to(dtype)
    w = (torch.randn(taps, channels, device="cuda", generator=g) * 0.5).to(dtype)
    state = torch.randn(len(t_sizes) + 1, max(taps - 1, 1), channels, device="cuda", generator=g).to(dtype)
    qsl = _i32(*[sum(t_sizes[:i]) for i in range(len(t_sizes) + 1)])
    lens = _i32(*[s + n for s, n in zip(starts, t_sizes)])
    slots = _i32(*range(1, len(t_sizes) + 1))
    seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(t_sizes)]).cuda()
    pos = torch.cat([torch.arange(s, s + n, dtype=torch.int32) for s, n in zip(starts, t_sizes)]).cuda()
    return x, w, state, slots, qsl, lens, seq, pos


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("channels,taps", [(24, 4), (20, 1), (264, 3), (40, 9)])
def test_short_conv_act(dtype, channels, taps):
    """Rows that start a sequence (the slot's contents must not show), rows that continue one, single rows that move
    their own state on, with and without SiLU."""
    hip = _hip()
    for t_sizes, starts in (([5, 1, 3, 1], [0, 7, 2, 0]), ([1, 1, 1], [4, 0, 1])):
        for silu in (True, False):
            x, w, state, slots, qsl, lens, seq, pos = _conv_case(dtype, t_sizes, starts, channels, taps, channels + taps)
            s1, s2 = state.clone(), state.clone()
            multi = max(t_sizes) > 1
            o1 = hip.short_conv_act(x, channels, w, s1, slots, qsl, lens, seq if multi else None, pos, silu, multi)
            o2 = torch_ref.short_conv_act(x, channels, w, s2, slots, qsl, lens, silu)
            _close(o1, o2, dtype, 4)
            for i, (start, n) in enumerate(zip(starts, t_sizes)):
                # the slot's rows that stand for positions of the sequence (rows for positions before its start are
                # never read; the kernel leaves them as they were)
                valid = min(start + n, taps - 1)
                if valid:
                    _close(s1[i + 1, taps - 1 - valid:], s2[i + 1, taps - 1 - valid:], dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("heads,kv,dim,vdim,taps,half", [(4, 2, 16, 8, 3, 4), (2, 1, 64, 64, 3, 32), (3, 3, 12, 20, 2, 6),
                                                          (2, 2, 32, 16, 4, 8), (2, 1, 24, 8, 1, 0)])
def test_conv_rotation_cache(dtype, heads, kv, dim, vdim, taps, half):
    """Convolution, no head norm, rotation of the first ``2 * half`` values of every q and k head, cache write."""
    hip = _hip()
    bs, nblk = 16, 6
    channels = heads * dim + kv * (dim + vdim)
    t_sizes, starts = [5, 1, 3], [0, 40, 17]
    x, w, state, slots, qsl, lens, seq, pos = _conv_case(dtype, t_sizes, starts, channels, taps, dim + taps)
    inv_freq = (10000.0 ** (-torch.arange(half, dtype=torch.float32) / max(half, 1))).cuda() if half else None
    slot_mapping = _i32(*[(2 * i + 1) * bs + (p % bs) for i, (s, n) in enumerate(zip(starts, t_sizes)) for p in range(s, s + n)])
    res = []
    for fn in (hip.conv_norm_cache, None):
        st = state.clone()
        kc = torch.zeros(nblk, kv, bs, dim, device="cuda", dtype=dtype)
        vc = torch.zeros(nblk, kv, bs // 8, vdim, 8, device="cuda", dtype=dtype)
        if fn is not None:
            q, _ = fn(x, w, st, slots, qsl, lens, seq, pos, heads, kv, dim, vdim, None, None, 1e-5, None, None, False, kc, vc,
                      slot_mapping, True, inv_freq)
        else:
            q, _ = torch_ref.conv_norm_cache(x, w, st, slots, qsl, lens, heads, kv, dim, vdim, None, None, 1e-5, None, None,
                                             False, kc, vc, slot_mapping, inv_freq, pos)
        res.append((q, kc, vc, st))
    for a, b in zip(*res):
        _close(a, b, dtype, 8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("heads,kv,dim,vdim", [(4, 2, 64, 64), (2, 2, 32, 16), (3, 1, 24, 8)])
def test_chunked_attention(dtype, heads, kv, dim, vdim):
    """Chunks of 20 positions over pages of 16: a prompt portion that crosses two chunk borders beside decoded rows at
    a chunk's first and last position, with a sink; both kernels (matrix cores where the shape allows)."""
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(dim)
    bs, nblk, chunk = 16, 12, 20
    kc = (torch.randn(nblk, kv, bs, dim, device="cuda", generator=g) * 0.5).to(dtype)
    vc = torch.randn(nblk, kv, bs // 8, vdim, 8, device="cuda", generator=g).to(dtype)
    table = torch.tensor([[3, 7, 1, 9, 0, 0], [2, 5, 8, 11, 4, 0], [6, 10, 0, 0, 0, 0]], dtype=torch.int32, device="cuda")
    sinks = torch.tensor([0.5, -1.0, 2.0, 0.0][:heads], device="cuda")
    for lens, rows in (([60, 80, 21], [1, 1, 1]), ([59, 70, 20], [45, 3, 20])):
        t = sum(rows)
        q = torch.randn(t, heads, dim, device="cuda", generator=g).to(dtype)
        qsl = _i32(*[sum(rows[:i]) for i in range(4)])
        seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(rows)]).cuda()
        pos = torch.cat([torch.arange(l - n, l, dtype=torch.int32) for l, n in zip(lens, rows)]).cuda()
        decode = max(rows) == 1
        got = hip.window_bias_attention(q, kc, vc, table, qsl, _i32(*lens), None if decode else seq, pos, dim ** -0.5, 0.0,
                                        chunk, 0, None, None, sinks, None, max(rows), None, chunk)
        want = torch_ref.window_bias_attention(q, kc, vc, table, qsl, _i32(*lens), dim ** -0.5, 0.0, chunk, 0, None, None,
                                               sinks, None, chunk)
        _close(got, want, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("heads,kv,dim,vdim", [(2, 1, 128, 128), (4, 2, 64, 64), (2, 2, 40, 24)])
def test_chunked_attention_over_many_pages(dtype, heads, kv, dim, vdim):
    """Chunks of 150 positions over shuffled pages of 16 and sequences of several chunks: prompt portions that start
    inside a chunk and cross one or two borders (whole key steps in front of a chunk's start are skipped), decoded rows
    at a chunk's last and first position and deep inside the third chunk."""
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(dim + 1)
    bs, chunk, per = 16, 150, 27
    nblk = 3 * per + 1
    kc = (torch.randn(nblk, kv, bs, dim, device="cuda", generator=g) * 0.4).to(dtype)
    vc = torch.randn(nblk, kv, bs // 8, vdim, 8, device="cuda", generator=g).to(dtype)
    table = (torch.randperm(nblk - 1, device="cuda", generator=g) + 1).to(torch.int32).view(3, per)
    sinks = torch.tensor([0.5, -1.0, 2.0, 0.0][:heads], device="cuda")
    for lens, rows in (([300, 301, 425], [1, 1, 1]), ([340, 151, 430], [200, 3, 137]), ([150, 432, 17], [150, 300, 17])):
        t = sum(rows)
        q = torch.randn(t, heads, dim, device="cuda", generator=g).to(dtype)
        qsl = _i32(*[sum(rows[:i]) for i in range(4)])
        seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(rows)]).cuda()
        pos = torch.cat([torch.arange(l - n, l, dtype=torch.int32) for l, n in zip(lens, rows)]).cuda()
        decode = max(rows) == 1
        got = hip.window_bias_attention(q, kc, vc, table, qsl, _i32(*lens), None if decode else seq, pos, dim ** -0.5, 0.0,
                                        chunk, 0, None, None, sinks, None, max(rows), None, chunk)
        want = torch_ref.window_bias_attention(q, kc, vc, table, qsl, _i32(*lens), dim ** -0.5, 0.0, chunk, 0, None, None,
                                               sinks, None, chunk)
        _close(got, want, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rank,rope,heads", [(16, 8, 2), (96, 16, 8), (20, 6, 3)])
def test_windowed_latent_rows(dtype, rank, rope, heads):
    """Neighbouring rotation pairs in the row and the query; a window of 19 over pages of 16 with sink and gate, for
    decoded rows and a prompt portion."""
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(rank)
    bs, nblk, nope, window = 16, 8, 12, 19
    t = 9
    q = torch.randn(t, heads, nope + rope, device="cuda", generator=g).to(dtype)
    q_lat = torch.randn(heads, t, rank, device="cuda", generator=g).to(dtype)
    wide = torch.randn(t, rank + rope + heads, device="cuda", generator=g).to(dtype)
    latent, gate = wide[:, :rank + rope], wide[:, rank + rope:]
    nw = torch.rand(rank, device="cuda", generator=g) + 0.5
    inv_freq = (100.0 ** (-torch.arange(rope // 2, dtype=torch.float32) / (rope // 2))).cuda()
    pos = torch.arange(30, 30 + t, dtype=torch.int32, device="cuda")
    slot_mapping = (2 * bs + pos).to(torch.int32)
    c1 = (torch.randn(nblk, 1, bs, rank + rope, device="cuda", generator=g) * 0.5).to(dtype)
    c2 = c1.clone()
    for inter in (True, False):
        o1 = hip.latent_prep(q, nope, q_lat, latent, nw, 1e-5, inv_freq, 1.0, pos, c1, slot_mapping, None, inter)
        o2 = torch_ref.latent_prep(q, nope, q_lat, latent, nw, 1e-5, inv_freq, 1.0, pos, c2, slot_mapping, None, inter)
        _close(o1, o2, dtype, 8)
        _close(c1, c2, dtype, 8)
    sinks = torch.randn(heads, device="cuda", generator=g)
    table = torch.tensor([[5, 1, 2, 7], [0, 3, 4, 6]], dtype=torch.int32, device="cuda")
    qf = torch.randn(t, heads, rank + rope, device="cuda", generator=g).to(dtype)
    for seq, lens in ((_i32(0, 0, 0, 0, 0, 1, 1, 1, 1), _i32(31, 32, 33, 34, 35, 18, 19, 20, 21)), (None, None)):
        if seq is None:                 # decoded rows: row t is sequence t
            table2 = table[:1].repeat(t, 1).contiguous()
            lens = _i32(1, 18, 19, 20, 21, 37, 38, 39, 64)
            got = hip.latent_row_attention(qf, c1, table2, None, lens, 0.2, rank, 64, window, sinks, gate)
            want = torch_ref.latent_row_attention(qf, c1, table2, None, lens, 0.2, rank, window, sinks, gate)
        else:
            got = hip.latent_row_attention(qf, c1, table, seq, lens, 0.2, rank, 64, window, sinks, gate)
            want = torch_ref.latent_row_attention(qf, c1, table, seq, lens, 0.2, rank, window, sinks, gate)
        _close(got, want, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("heads,qk,dim,vdim", [(4, 4, 32, 32), (4, 2, 8, 12), (2, 1, 128, 128), (3, 3, 72, 24), (1, 1, 200, 8)])
def test_gated_delta_rule(dtype, heads, qk, dim, vdim):
    """Three sequences in one launch (a fresh prompt portion, a continuing one, a decoded row) against the reference
    recurrence; the states of other slots stay as they were."""
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(dim)
    rows, starts = [13, 6, 1], [0, 9, 50]
    t = sum(rows)
    x = (torch.randn(t, 2 * qk * dim + heads * vdim + 4, device="cuda", generator=g) * 0.8).to(dtype)
    wide = torch.randn(t, heads + heads * dim, device="cuda", generator=g).to(dtype)
    beta, dtr = wide[:, :heads], wide[:, heads:]
    dt_bias = torch.randn(heads * dim, device="cuda", generator=g) * 0.5
    a_log = torch.randn(heads, device="cuda", generator=g) - 1.0
    state = torch.randn(5, heads, dim, vdim, device="cuda", generator=g) * 0.3
    s1, s2 = state.clone(), state.clone()
    qsl, lens, slots = _i32(0, 13, 19, 20), _i32(*[s + n for s, n in zip(starts, rows)]), _i32(3, 0, 4)
    o1 = hip.gated_delta_rule(x, heads, qk, dim, vdim, beta, dtr, dt_bias, a_log, s1, slots, qsl, lens, 1e-6, 13)
    o2 = torch_ref.gated_delta_rule(x, heads, qk, dim, vdim, beta, dtr, dt_bias, a_log, s2, slots, qsl, lens, 1e-6)
    _close(o1, o2, torch.float32, 8)                   # (inputs are read in the same type: the arithmetic is fp32 in both)
    _close(s1, s2, torch.float32, 8)
    assert torch.equal(s1[1], state[1]) and torch.equal(s1[2], state[2])


@pytest.mark.parametrize("window", [0, 19, 70])
def test_windowed_latent_rows_on_the_matrix_cores(window):
    """Latent rows of 64 + 32 values kept as rows and as V^T fragments: the matrix-core kernels with a window, sinks
    and a gate (one token per workgroup, four consecutive tokens per workgroup, split keys) against the reference
    over the rows."""
    hip = _hip()
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(window)
    rank, rope, heads, bs, nblk = 64, 32, 5, 16, 20
    n = 150
    table = torch.randperm(nblk, generator=torch.Generator().manual_seed(1))[:10].to(torch.int32).view(1, -1).cuda()
    rows_c = torch.zeros(nblk, 1, bs, rank + rope, device="cuda", dtype=dtype)
    frags = torch.zeros(nblk, 1, rank // 16, bs // 8, 16, 8, device="cuda", dtype=dtype)
    latent = (torch.randn(n, rank + rope, device="cuda", generator=g) * 0.7).to(dtype)
    q = torch.randn(n, heads, 16 + rope, device="cuda", generator=g).to(dtype)
    q_lat = torch.randn(heads, n, rank, device="cuda", generator=g).to(dtype)
    nw = torch.rand(rank, device="cuda", generator=g) + 0.5
    inv_freq = (100.0 ** (-torch.arange(rope // 2, dtype=torch.float32) / (rope // 2))).cuda()
    pos = torch.arange(n, dtype=torch.int32, device="cuda")
    slots = (table[0, (pos // bs).long()] * bs + pos % bs).to(torch.int32)
    hip.latent_prep(q, 16, q_lat, latent, nw, 1e-5, inv_freq, 1.0, pos, rows_c, slots, frags, True)
    sinks = torch.randn(heads, device="cuda", generator=g)
    wide = torch.randn(n, heads + 3, device="cuda", generator=g).to(dtype)
    gate = wide[:, 3:]
    qf = torch.randn(n, heads, rank + rope, device="cuda", generator=g).to(dtype)
    # a prompt portion: rows 0 .. 39 are positions 110 .. 149 of the sequence
    t = 40
    seq, lens = torch.zeros(t, dtype=torch.int32, device="cuda"), torch.arange(111, 151, dtype=torch.int32, device="cuda")
    want = torch_ref.latent_row_attention(qf[:t], rows_c, table, seq, lens, 0.15, rank, window, sinks, gate[:t])
    for mode, splits in ((1, None), (1, 2), (0, 1), (0, 3)):
        got = hip.mla_attention(qf[:t], rows_c, frags, table, seq, lens, 0.15, 150, None, splits, mode, True, window,
                                sinks, gate[:t])
        _close(got, want, dtype, 2)
    # decoded rows of sequences of other lengths
    lens = _i32(1, 2, 18, 19, 20, 21, 64, 65, 150)
    table9 = table.repeat(9, 1).contiguous()
    want = torch_ref.latent_row_attention(qf[:9], rows_c, table9, None, lens, 0.15, rank, window, sinks, gate[:9])
    for splits in (None, 1, 2):
        got = hip.mla_attention(qf[:9], rows_c, frags, table9, None, lens, 0.15, 150, None, splits, 0, True, window, sinks,
                                gate[:9])
        _close(got, want, dtype, 2)
