"""Nalasun through the framework (loader, scheduler, block and state-slot bookkeeping, model runner, kernels on the
GPU / reference ops on the CPU) against the plain float64 model of ``tests/nalasun_oracle.py``.

Every test builds its own small configuration and random weights (stored as bfloat16, so the oracle and the framework
read the same numbers).  The schedules go through ``EngineCore.step_forced`` and generation goes through
``LLM.generate``.  The CPU tests run in float32; the GPU tests run the HIP kernels in float32 (tight tolerance: an index
that is one off shows) and in bfloat16 (with routers made decisive, see ``model_dir``).
"""
import json
import math
import os

import numpy as np
import pytest
import torch

import nalasun_oracle as oracle
from test_tavulix import portions, run_schedule, tokens_for

F64 = torch.float64


# ------------------------------------------------------------------------------------------------ models
def attention(heads, kv, dim, scale, temp=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def delta(heads, kv, dim, vdim, conv, mlp=None):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp}


def ssm(heads, vdim, state, groups, norm_groups, conv, mlp=None):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                        "norm_groups": norm_groups, "conv": conv}, "mlp": mlp}


def moe(experts, top, ff, scale=1.0, shared=0):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale},
            "shared": {"ff": shared} if shared else None}


def config(layers, width=48, vocab=97, eps=1e-5, taps=3, positions=400):
    c = {"architecture": "Nalasun", "vocab": vocab, "width": width, "max_positions": positions, "norm": {"eps": eps},
         "layers": layers}
    if taps:
        c["canon"] = {"taps": taps}
    return c


# (the widths of the two low-rank projections of a channel_delta mixer are sizes only the tensors state)
RANKS = {"varied": (6, 10), "degenerate": (3, 3), "paged": (5, 7), "wide": (8, 8), "uneven": (5, 9)}

CONFIGS = {
    # every layer of another shape and kind, a recurrent layer first; value heads sharing q / k heads; B / C groups
    # shared by heads; a layer without feed-forward; a block without shared expert; a shared expert wider than the
    # routed ones; temperatures that step every few tokens
    "varied": config([
        ssm(4, 12, 10, 2, 2, 4, moe(5, 2, 24, 1.5, 40)),
        attention(4, 2, 16, 0.2, (0.3, 5), moe(4, 3, 16, 0.7)),
        delta(4, 2, 8, 12, 4, None),
        attention(6, 3, 8, 0.3, (0.5, 16), moe(5, 2, 24, 2.0, 16)),
        ssm(2, 20, 6, 1, 1, 2, None)]),
    # values a model can make equal or one: one head, kv heads = heads, one B / C group per head, one norm group and
    # one per head, one tap everywhere and no input convolution at all, top 1 of 1 expert and top = experts, a router
    # scale of exactly one, no temperature
    "degenerate": config([
        attention(1, 1, 16, 0.25, None, moe(1, 1, 16)),
        ssm(2, 8, 4, 2, 2, 1, moe(3, 3, 8, 1.0, 8)),
        delta(1, 1, 8, 8, 1, None),
        attention(2, 2, 8, 0.35, None, None)], width=32, vocab=50, taps=0),
    # sequences over several pages of 16 tokens; attention first
    "paged": config([
        attention(4, 1, 16, 0.22, (0.4, 33), moe(6, 2, 32, 1.25, 32)),
        delta(4, 2, 16, 16, 3, moe(4, 2, 32, 1.0, 0)),
        ssm(4, 16, 16, 2, 4, 4, None),
        attention(2, 2, 32, 0.15, (0.2, 7), None)], width=64, taps=4),
    # sizes the 16-bit kernels' 16-byte and matrix-core paths take (head sizes of 32 / 64, a width of 128)
    "wide": config([
        delta(4, 4, 32, 32, 4, moe(4, 2, 64, 1.5, 64)),
        attention(4, 2, 64, 0.11, (0.3, 20), moe(4, 2, 64, 1.5, 64)),
        ssm(4, 32, 32, 1, 2, 4, None),
        attention(8, 2, 32, 0.16, (0.3, 64), None)], width=128, taps=2),
    # a width, a vocabulary and sizes that are no multiples of 8 (no 16-byte access fits a 16-bit row); one tap of
    # input convolution
    "uneven": config([
        ssm(3, 10, 7, 3, 1, 3, moe(5, 2, 30, 0.9, 22)),
        attention(3, 1, 20, 0.2, (0.35, 9), None),
        delta(3, 3, 12, 20, 2, moe(3, 1, 26, 1.7, 0))], width=100, vocab=211, taps=1),
}


def random_weights(cfg, seed, ranks):
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]
    taps = (cfg.get("canon") or {}).get("taps") or 0

    def rnd(*shape, lo=-1.0, hi=1.0):
        return lo + (hi - lo) * torch.rand(shape, generator=g)

    def proj(rows, cols, gain=1.0):
        return rnd(rows, cols) * gain * (3.0 / cols) ** 0.5

    w = {"embed": rnd(cfg["vocab"], width), "pos": rnd(cfg["max_positions"], width, lo=-0.5, hi=0.5),
         "final.norm": rnd(width, lo=0.6, hi=1.4)}
    for i, spec in enumerate(cfg["layers"]):
        m, p, q = spec["mixer"], f"l{i}.", f"l{i}.mix."
        w[p + "norm1"] = rnd(width, lo=0.6, hi=1.4)
        if taps:
            w[p + "canon1"] = rnd(width, taps, lo=-0.5, hi=0.5)
        if spec["type"] == "attention":
            heads, kv, dim = m["heads"], m["kv_heads"], m["dim"]
            w[q + "q"], w[q + "q.b"], w[q + "q.norm"] = proj(heads * dim, width), rnd(heads * dim, lo=-0.3, hi=0.3), rnd(heads * dim, lo=0.5, hi=1.5)
            w[q + "k"], w[q + "k.b"], w[q + "k.norm"] = proj(kv * dim, width), rnd(kv * dim, lo=-0.3, hi=0.3), rnd(kv * dim, lo=0.5, hi=1.5)
            w[q + "r1"], w[q + "r2"] = rnd(heads, lo=0.0, hi=1.2), rnd(heads, lo=0.05, hi=0.6)
            w[q + "talk"] = torch.eye(heads) + rnd(heads, heads, lo=-0.4, hi=0.4)
            w[q + "o"] = proj(width, heads * dim)
        elif spec["type"] == "channel_delta":
            heads, kv, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for nm, rows in (("q", kv * dim), ("k", kv * dim), ("v", heads * vdim)):
                w[q + nm], w[q + nm + ".conv"] = proj(rows, width, 2.0), rnd(rows, m["conv"])
            w[q + "b"], w[q + "A_log"], w[q + "norm"] = proj(heads, width, 2.0), rnd(heads, lo=-2.5, hi=0.5), rnd(vdim, lo=0.6, hi=1.4)
            w[q + "a1"], w[q + "a2"] = proj(ranks[0], width, 2.0), proj(heads * dim, ranks[0], 2.0)
            w[q + "dt_bias"] = rnd(heads * dim, lo=-1.0, hi=1.0)
            w[q + "g1"], w[q + "g2"] = proj(ranks[1], width, 2.0), proj(heads * vdim, ranks[1], 2.0)
            w[q + "o"] = proj(width, heads * vdim)
        else:
            heads, vdim, n, groups = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = heads * vdim, heads * vdim + 2 * groups * n
            w[q + "in"] = proj(2 * inner + 2 * groups * n + heads, width, 1.5)
            w[q + "conv"], w[q + "conv.b"] = rnd(ch, m["conv"], lo=-0.7, hi=0.7), rnd(ch, lo=-0.3, hi=0.3)
            w[q + "dt_bias"], w[q + "A_log"], w[q + "D"] = rnd(heads, lo=-3.0, hi=0.0), rnd(heads, lo=-3.0, hi=0.5), rnd(heads, lo=0.3, hi=1.0)
            w[q + "norm"], w[q + "o"] = rnd(inner, lo=0.6, hi=1.4), proj(width, inner)
        mlp = spec["mlp"]
        if mlp:
            w[p + "norm2"] = rnd(width, lo=0.6, hi=1.4)
            names = [(f"e{e}", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                names.append(("shared", mlp["shared"]["ff"]))
            for nm, ff in names:
                w[f"{p}mlp.{nm}.gate"], w[f"{p}mlp.{nm}.up"] = proj(ff, width, 2.0), proj(ff, width, 1.5)
                w[f"{p}mlp.{nm}.down"] = proj(width, ff)
            w[p + "mlp.router"] = proj(mlp["router"]["experts"], width, 3.0)
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


_MODELS = {}


def model_dir(name, tmp_path_factory, dtype="float32"):
    """The model's folder, configuration and weights.  For bfloat16 runs the routers are made decisive: the design's
    router has no bias, so the residual stream gets a constant of its own - coordinate 0 of every position vector is
    3, of every token vector 0, and no mixer or expert writes to it - and every router reads that coordinate only,
    with multipliers 1.5 apart in a random order.  The order of the scores is then the same for every token whatever rounding does to the logits,
    while the scores, which are the weights, still differ from token to token.  In bfloat16 the router's input carries
    the rounding of every layer before it, and a close call that falls the other way swaps a whole expert; the float32
    runs keep the free-running routers."""
    decisive = dtype != "float32"
    if (name, decisive) not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]
        w = random_weights(cfg, sum(map(ord, name)), RANKS[name])
        if decisive:
            g = torch.Generator().manual_seed(11)
            w["pos"][:, 0], w["embed"][:, 0] = 3.0, 0.0
            for k in [k for k in w if k.endswith(".o") or k.endswith(".down")]:
                w[k][0] = 0.0
            for k in [k for k in w if k.endswith(".router")]:
                experts = w[k].shape[0]
                w[k] = torch.zeros_like(w[k])
                w[k][:, 0] = ((torch.randperm(experts, generator=g).float() - (experts - 1) / 2) * 1.5).to(torch.bfloat16)
                w[k[:-len("mlp.router")] + "norm2"][0] = 1.0
        d = tmp_path_factory.mktemp("nalasun_" + name)
        save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[(name, decisive)] = (str(d), cfg, w)
    return _MODELS[(name, decisive)]


_ORACLE = {}


def oracle_logits(name, cfg, w, tokens, single=False):
    """The float64 model's logits; ``single``: the same equations evaluated in float32."""
    key = (name, id(w), tuple(tokens), single)
    if key not in _ORACLE:
        kind = torch.float32 if single else torch.float64
        saved = oracle.F64, oracle.f64
        oracle.F64, oracle.f64 = kind, (lambda t: t.to(kind))
        try:
            _ORACLE[key] = oracle.forward(cfg, w, list(tokens)).double().numpy()
        finally:
            oracle.F64, oracle.f64 = saved
    return _ORACLE[key]


def check(got, name, cfg, w, reqs, tol):
    """Every row the run produced against the oracle.  The recurrent layers' outputs are normed, so at a position
    where such an output nearly cancels, the rounding of its inputs is multiplied up, by thousands now and then.  How
    much a row multiplies rounding is measured, not guessed: the oracle's own equations evaluated in float32 differ
    from float64 by some ``e32`` at that row (a few 1e-6 where nothing cancels), and the row is allowed ``8 e32`` in
    float32 and ``2^14 e32`` in bfloat16 where that is more than the tolerance.  A wrong index or a lost state shows
    in many rows, none of them of that kind."""
    assert got
    room = 8.0 if tol < 1e-2 else 16384.0
    over = []
    for (rid, p), row in got.items():
        want = oracle_logits(name, cfg, w, reqs[rid])[p]
        e32 = float(np.abs(oracle_logits(name, cfg, w, reqs[rid], single=True)[p] - want).max())
        ratio = float(np.abs(row - want).max()) / max(tol, room * e32)
        if ratio > 1.0:
            over.append((ratio, rid, p, e32))
    over.sort(reverse=True)
    # (in bfloat16 a row in fifty may lie outside, by a factor of three at most: the tolerance is a typical worst row)
    assert not over or over[0][0] <= 3.0, over[:5]
    assert len(over) <= max(1, len(got) // 50), over[:5]


DEVICES = [pytest.param("cpu", "float32", 2e-4, id="cpu-f32"),
           pytest.param("cuda", "float32", 2e-4, id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", 0.5, id="gpu-bf16", marks=pytest.mark.gpu)]


# ------------------------------------------------------------------------------------------------ schedules
@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_first_tokens(name, device, dtype, tol, tmp_path_factory, tmp_path):
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    reqs = {"a": tokens_for(cfg, 90, 1), "b": tokens_for(cfg, 1, 2), "c": tokens_for(cfg, 2, 3)}
    steps = [[(r, t, list(range(len(t)))), {"end": [r]}] for r, t in reqs.items()]
    got = run_schedule(path, steps, dtype, device, max_tokens=128, tmp=tmp_path)
    assert len(got) == 93
    check(got, name, cfg, w, reqs, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_residual_stream_after_every_layer(device, dtype, tol, tmp_path_factory):
    if dtype != "float32":
        pytest.skip("the per-layer comparison is the float32 one")
    import types
    from vllm_distributed_amd.entrypoints import trace_replay
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
    toks = tokens_for(cfg, 37, 8)
    args = types.SimpleNamespace(model=path, dtype=dtype, out="", max_tokens=64, max_seqs=2, device=device,
                                 block_size=16, enforce_eager=True)
    core = trace_replay.make_core(args)
    try:
        from vllm_distributed_amd.engine.request import Request
        from vllm_distributed_amd.sampling_params import SamplingParams
        model = core.executor.driver.worker.model_runner.model
        model.trace_residual = []
        core.add_request(Request("r", toks, SamplingParams(temperature=0.0, max_tokens=None, score_only=True, ignore_eos=True)))
        core.step_forced({"r": len(toks)}, {})
        got = [t.cpu().double() for t in model.trace_residual]
    finally:
        core.shutdown()
    want = []
    oracle.forward(cfg, w, toks, want)
    assert len(got) == len(want) == 5
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item()), i


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", ["varied", "paged", "wide"])
def test_prefill_then_long_token_by_token_decoding(name, device, dtype, tol, tmp_path_factory, tmp_path):
    """A prompt, then 150 tokens one at a time: recurrent states and convolution tails are carried through 150
    single-row steps, the cache grows over several pages, every temperature step is passed by decoded tokens."""
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    toks = tokens_for(cfg, 190, 4)
    got = run_schedule(path, portions(toks, [40, 1], "r"), dtype, device, max_tokens=192, tmp=tmp_path)
    assert len(got) == 190
    check(got, name, cfg, w, {"r": toks}, tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 0.5)])
@pytest.mark.parametrize("name", ["paged", "wide"])
def test_pages_of_64_tokens(name, dtype, tol, tmp_path_factory, tmp_path):
    """The page size a GPU engine uses by default: two requests in turn, portions that end inside, at and just
    behind a page's border, then single rows across the next border."""
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    a, b = tokens_for(cfg, 150, 60), tokens_for(cfg, 70, 61)
    steps = [[("a", a[:63], [0, 62])], [("a", a[63:64], [0]), ("b", b[:64], [63])], [("a", a[64:66], [0, 1]), ("b", b[64:65], [0])],
             [("a", a[66:127], [60]), ("b", b[65:70], [4]), {"end": ["b"]}]]
    steps += [[("a", a[i:i + 1], [0])] for i in range(127, 150)]
    steps[-1].append({"end": ["a"]})
    got = run_schedule(path, steps, dtype, "cuda", max_tokens=256, block_size=64, tmp=tmp_path)
    assert len(got) == 2 + 1 + 1 + 2 + 1 + 1 + 1 + 23
    check(got, name, cfg, w, {"a": a, "b": b}, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7, 1, 16, 17, 2, 2, 31, 5], [1], [64, 2, 1]])
def test_portions_of_any_size(sizes, device, dtype, tol, tmp_path_factory, tmp_path):
    """Portions cut inside pages, convolution tails and temperature steps, down to two tokens and one."""
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
    toks = tokens_for(cfg, 75 if sizes != [1] else 40, 5)
    got = run_schedule(path, portions(toks, sizes, "r"), dtype, device, max_tokens=128, tmp=tmp_path)
    assert len(got) == len(toks)
    check(got, "varied", cfg, w, {"r": toks}, tol)


@pytest.mark.parametrize("eager", [False, True])
@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_mixed_batches_reuse_pages_and_slots(device, dtype, tol, eager, tmp_path_factory, tmp_path):
    """Seven unequal requests through three sequence slots and a pool of 10 pages: portions of prompts beside single
    tokens, requests that sit steps out, state slots and pages handed on as requests end (a new owner must not see
    what the old one left); every row against the request run alone by the oracle."""
    if eager and device == "cpu":
        pytest.skip("graphs exist on the GPU only")
    path, cfg, w = model_dir("paged", tmp_path_factory, dtype)
    reqs = {f"q{i}": tokens_for(cfg, n, 10 + i) for i, n in enumerate([50, 33, 1, 47, 20, 48, 9])}
    at = {r: 0 for r in reqs}
    pattern = {"q0": [7, 1, 1, 2, 30, 1], "q1": [2, 16, 1, 1, 1], "q2": [1], "q3": [17, 1, 15, 1], "q4": [1, 1, 5],
               "q5": [30, 2, 1], "q6": [2, 1]}
    waiting, live, steps, turn = list(reqs), [], [], 0
    while waiting or live:
        while waiting and len(live) < 3 and \
                sum(-(-len(reqs[r]) // 64) * 64 for r in live + waiting[:1]) <= 160:
            live.append(waiting.pop(0))
        step, ended = [], []
        for k, r in enumerate(list(live)):
            if (turn + k) % 4 == 3 and len(live) > 1:
                continue                                    # sits this step out
            sizes = pattern[r]
            n = min(sizes[min(at[r] and (turn % len(sizes)), len(sizes) - 1)], len(reqs[r]) - at[r])
            step.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == len(reqs[r]):
                ended.append(r)
                live.remove(r)
        if step:
            steps.append(step + ([{"end": ended}] if ended else []))
        turn += 1
    got = run_schedule(path, steps, dtype, device, max_tokens=160, max_seqs=3, eager=eager, tmp=tmp_path)
    assert len(got) == sum(len(t) for t in reqs.values())
    check(got, "paged", cfg, w, reqs, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_batch_rows_equal_single_runs(device, dtype, tol, tmp_path_factory, tmp_path):
    """The same rows run alone and inside a batch of unequal neighbours agree far inside the oracle tolerance."""
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
    a, b, c = tokens_for(cfg, 30, 20), tokens_for(cfg, 11, 21), tokens_for(cfg, 64, 22)
    alone = run_schedule(path, portions(a, [13, 1], "a"), dtype, device, max_tokens=64, tmp=tmp_path / "x")
    steps = [[("c", c[:50], []), ("a", a[:13], list(range(13))), ("b", b[:2], [])]]
    for i in range(13, 30):
        step = [("a", a[i:i + 1], [0])]
        if i < 22:
            step.append(("b", b[i - 11:i - 10], []))
        if i < 27:
            step.insert(0, ("c", c[50 + i - 13:51 + i - 13], []))
        steps.append(step)
    both = run_schedule(path, steps, dtype, device, max_tokens=192, tmp=tmp_path / "y")
    worst = sorted(float(np.abs(alone[("a", p)] - both[("a", p)]).max()) for p in range(30))
    assert worst[-1 if dtype == "float32" else -2] <= (1e-4 if dtype == "float32" else 0.2), worst[-3:]


# --------------------------------------------------------------------------- mechanisms alone, made to show
OP_DEVICES = [pytest.param("cpu", "float32", id="cpu-f32"),
              pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
              pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]


def i32(device, *values):
    return torch.tensor(list(values), dtype=torch.int32, device=device)


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_the_state_space_scan_remembers_far_tokens_and_stale_slots_do_not_show(device, dtype):
    """Token 0 writes a value along one state channel; 300 tokens later a read-out along that channel returns it,
    shrunk by the decays in between, from a head that keeps and nothing from a head that forgets; the tokens between
    write next to nothing (tiny step sizes).  The sequence runs in portions of many sizes through a slot another
    sequence left full, and the whole is compared with the token-by-token float64 recurrence."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    heads, groups, vdim, n_state, n = 2, 1, 8, 6, 301
    g = torch.Generator().manual_seed(3)
    x = torch.randn(n, heads, vdim, generator=g) * 0.05
    b = torch.randn(n, groups, n_state, generator=g) * 0.02
    c = torch.randn(n, groups, n_state, generator=g) * 0.02
    b[0, 0, 2], c[n - 1, 0, 2] = 3.0, 2.0
    x[0, :, 1] = 4.0
    step_in = torch.full((n, heads), -6.0)                     # softplus(-6) ~ 0.0025: next to no write, slow decay
    step_in[0] = 3.0
    a_log = torch.tensor([math.log(0.4), math.log(60.0)])      # head 0 keeps (~ 0.999 per token), head 1 forgets
    dt_bias, skip = torch.zeros(heads), torch.tensor([0.5, 0.25])
    rows = torch.cat([x.reshape(n, -1), b.reshape(n, -1), c.reshape(n, -1)], 1).to(dt)
    step_in = step_in.to(dt)
    rf = rows.double()
    xs, bs_, cs_ = rf[:, :heads * vdim].view(n, heads, vdim), rf[:, heads * vdim:heads * vdim + n_state], rf[:, heads * vdim + n_state:]
    want, _ = oracle.ssm_heads(xs, bs_.view(n, 1, n_state).repeat(1, heads, 1), cs_.view(n, 1, n_state).repeat(1, heads, 1),
                               oracle.softplus(step_in.double()), torch.exp(a_log.double()), skip.double())
    far = want[n - 1, 0, 1] - 0.5 * xs[n - 1, 0, 1]
    d0 = float(oracle.softplus(torch.tensor(3.0, dtype=F64)))
    assert abs(float(far) - d0 * 3.0 * 4.0 * 2.0 * math.exp(-0.4 * 300 * math.log1p(math.exp(-6.0)))) < 0.5
    assert abs(float(want[n - 1, 1, 1] - 0.25 * xs[n - 1, 1, 1])) < 0.05
    state = torch.full((3, heads, n_state, vdim), 7.0, device=device)              # what an earlier owner left
    out, at, sizes = [], 0, [1, 2, 64, 17, 1, 1, 100, 3, 2]
    for i in range(100):
        m = min(sizes[i % len(sizes)], n - at)
        if m == 0:
            break
        out.append(ops.selective_scan(rows[at:at + m].to(device), step_in[at:at + m].to(device), heads, groups, vdim,
                                      n_state, a_log.to(device), dt_bias.to(device), skip.to(device), state,
                                      i32(device, 2), i32(device, 0, m), i32(device, at + m)).cpu())
        at += m
    got = torch.cat(out).view(n, heads, vdim).double()
    assert (got - want).abs().max().item() < (1e-5 if dtype == "float32" else 2e-3) * float(want.abs().max())
    assert float(state[0].min()) == 7.0 and float(state[1].max()) == 7.0


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
@pytest.mark.parametrize("n_state,vdim,heads,groups", [(24, 20, 3, 1), (32, 32, 4, 4), (96, 40, 2, 2), (160, 16, 1, 1),
                                                       (10, 7, 2, 2), (66, 70, 2, 1)])
def test_state_space_scan_sizes(device, dtype, n_state, vdim, heads, groups):
    """State sizes on both sides of every tiling of the scan kernel, heads sharing B / C groups, two sequences in one
    call (one continuing from a state, one starting)."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(n_state)
    n = [9, 5]
    t = sum(n)
    inner = heads * vdim
    rows = (torch.randn(t, inner + 2 * groups * n_state, generator=g) * 0.7).to(dt)
    step_in = torch.randn(t, heads, generator=g).to(dt)
    dt_bias, a_log, skip = torch.randn(heads, generator=g) - 1.0, torch.randn(heads, generator=g) - 1.0, torch.rand(heads, generator=g)
    s0 = torch.randn(heads, n_state, vdim, generator=g) * 0.3
    state = torch.full((4, heads, n_state, vdim), 5.0)
    state[1] = s0
    state = state.to(device)
    got = ops.selective_scan(rows.to(device), step_in.to(device), heads, groups, vdim, n_state, a_log.to(device),
                             dt_bias.to(device), skip.to(device), state, i32(device, 1, 3), i32(device, 0, n[0], t),
                             i32(device, 20 + n[0], n[1])).cpu().double().view(t, heads, vdim)
    rf = rows.double()
    rep = heads // groups
    x = rf[:, :inner].view(t, heads, vdim)
    b = rf[:, inner:inner + groups * n_state].view(t, groups, n_state).repeat_interleave(rep, 1)
    c = rf[:, inner + groups * n_state:].view(t, groups, n_state).repeat_interleave(rep, 1)
    step = oracle.softplus(step_in.double() + dt_bias.double())
    rate = torch.exp(a_log.double())
    w0, e0 = oracle.ssm_heads(x[:n[0]], b[:n[0]], c[:n[0]], step[:n[0]], rate, skip.double(), s0.double())
    w1, e1 = oracle.ssm_heads(x[n[0]:], b[n[0]:], c[n[0]:], step[n[0]:], rate, skip.double())
    tol = 2e-4 if dtype == "float32" else 2e-3
    scale = max(1.0, float(torch.cat([w0, w1]).abs().max()))
    assert (got - torch.cat([w0, w1])).abs().max().item() < tol * scale
    assert (state[1].cpu().double() - e0).abs().max().item() < tol * scale
    assert (state[3].cpu().double() - e1).abs().max().item() < tol * scale
    assert float(state[0].min()) == 5.0 and float(state[2].max()) == 5.0


def _paged(keys, vals, table, nblk, bs, dt):
    n, hkv, dim = keys.shape
    kc, vc = torch.zeros(nblk, hkv, bs, dim), torch.zeros(nblk, hkv, bs // 8, vals.shape[2], 8)
    for j in range(n):
        blk, off = int(table[0, j // bs]), j % bs
        kc[blk, :, off], vc[blk, :, off // 8, :, off % 8] = keys[j], vals[j]
    return kc.to(dt), vc.to(dt)


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
@pytest.mark.parametrize("dim", [8, 32])
def test_one_key_stands_out_far_back_and_at_page_borders(device, dtype, dim):
    """Key rows and values in shuffled pages of 16; the query is aimed at ONE key among hundreds: every query head's
    output on every value head is that key's value in that value head - far back, on both sides of page borders, the
    first token, the row itself - and never a key behind the row; as a decoded row and as the last row of a prompt
    portion.  With the distance bias on, a far key's weight falls as ``(1 + r2 d)^-r1``, in closed form."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    n, bs, hq, hkv = 330, 16, 4, 2
    g = torch.Generator().manual_seed(dim)
    nblk = -(-n // bs) + 2
    table = torch.randperm(nblk, generator=g)[:-(-n // bs)].to(torch.int32).view(1, -1)
    keys = torch.randn(n, hkv, dim, generator=g) * 0.3
    vals = torch.randn(n, hkv, dim, generator=g)
    aim = torch.zeros(dim)
    aim[1] = 3.0                                           # the target's key: far longer than any other key
    for pos in (329, 200, 47, 16, 15, 0):
        for target in sorted({0, 1, pos, pos - 1, pos // bs * bs, pos // bs * bs - 1, 15, 16, pos + 1, pos // 2}):
            if target < 0 or target >= n:
                continue
            kt = keys.clone()
            kt[target, :] = aim
            kc, vc = _paged(kt, vals, table, nblk, bs, dt)
            for rows in (1, min(9, pos + 1)):
                q = torch.randn(rows, hq, dim, generator=g) * 0.01
                q[-1] = aim * 20 / 3.0
                positions = torch.arange(pos - rows + 1, pos + 1, dtype=torch.int32, device=device)
                o = ops.crossed_bias_attention(q.to(dt).to(device), kc.to(device), vc.to(device), table.to(device),
                                               i32(device, 0, rows), i32(device, pos + 1),
                                               None if rows == 1 else torch.zeros(rows, dtype=torch.int32, device=device),
                                               positions, 1.0, None, None, rows)
                assert tuple(o.shape) == (rows, hq, hkv, dim) and o.dtype == torch.float32
                for c in range(hkv):
                    want = vc[table[0, target // bs], c, (target % bs) // 8, :, target % 8].float() if target < n else None
                    for h in range(hq):
                        hit = (o[-1, h, c].cpu() - want).abs().max().item() < 0.05
                        assert hit == (target <= pos), (target, pos, rows, h, c)
    # two visible keys with equal q.k: the bias alone decides, weight ratio (1 + r2 d)^-r1
    kt = torch.zeros(40, hkv, dim)
    kt[3, :, 0], kt[39, :, 0] = 1.0, 1.0
    vt = torch.zeros(40, hkv, dim)
    vt[3, :, 0], vt[39, :, 1] = 1.0, 1.0
    kt[:, :, 2] = -50.0                                    # every other key far below (the query has a 1 there)
    kt[3, :, 2] = kt[39, :, 2] = 0.0
    tb = torch.arange(3, dtype=torch.int32).view(1, -1)
    kc, vc = _paged(kt, vt, tb, 3, bs, dt)
    q = torch.zeros(1, hq, dim)
    q[..., 0], q[..., 2] = 1.0, 1.0
    r1, r2 = torch.tensor([0.0, 0.5, 1.0, 2.0]), torch.tensor([1.0, 0.25, 0.5, 0.125])
    o = ops.crossed_bias_attention(q.to(dt).to(device), kc.to(device), vc.to(device), tb.to(device), i32(device, 0, 1),
                                   i32(device, 40), None, i32(device, 39), 1.0, r1.to(device), r2.to(device), 1).cpu()
    for h in range(hq):
        far = (1.0 + float(r2[h]) * 36.0) ** -float(r1[h])
        assert abs(float(o[0, h, 0, 0]) - far / (1.0 + far)) < 2e-3, h


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_values_are_the_projected_keys_and_the_temperature_steps(device, dtype):
    """``joint_norm_cache``: q and k are normed over ALL their heads at once (not head by head), the key rows get the
    normed keys and the values the projection itself, and the query's factor steps exactly where
    ``floor((p + 1) / every)`` does (positions every - 2, every - 1, 2 every - 2, 2 every - 1)."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    heads, kv, dim, every, coef, bs = 4, 2, 8, 6, 0.5, 16
    g = torch.Generator().manual_seed(4)
    pos = [0, 4, 5, 6, 10, 11, 12, 35]
    t = len(pos)
    x = torch.randn(t, (heads + kv) * dim, generator=g)
    x[:, :dim] *= 6.0                                     # one head much larger: a per-head norm would flatten it
    x = x.to(dt)
    qw, kw = torch.rand(heads * dim, generator=g) + 0.5, torch.rand(kv * dim, generator=g) + 0.5
    kc, vc = torch.zeros(3, kv, bs, dim, dtype=dt, device=device), torch.zeros(3, kv, bs // 8, dim, 8, dtype=dt, device=device)
    slots = [17, 3, 40, 41, 9, 47, 32, 0]
    q = ops.joint_norm_cache(x.to(device), heads, kv, dim, qw.to(device), kw.to(device), 1e-5, i32(device, *pos), coef,
                             every, kc, vc, i32(device, *slots)).float().cpu().double().view(t, heads * dim)
    xf = x.double()
    qf, kf = xf[:, :heads * dim], xf[:, heads * dim:]
    temp = oracle.q_temperature(torch.tensor(pos), coef, every)
    assert [round(float(v), 6) for v in temp[[1, 2, 5, 6]]] == [1.0, round(1 + coef * math.log(2), 6),
                                                                round(1 + coef * math.log(3), 6), round(1 + coef * math.log(3), 6)]
    want_q = oracle.unit_rms(qf, 1e-5) * qw.double() * temp.view(-1, 1)
    tol = 1e-5 if dtype == "float32" else 0.03
    assert (q - want_q).abs().max().item() < tol * float(want_q.abs().max())
    per_head = oracle.unit_rms(qf.view(t, heads, dim), 1e-5).reshape(t, -1) * qw.double() * temp.view(-1, 1)
    assert (q - per_head).abs().max().item() > 0.3                                  # (the other reading is far away)
    want_k = oracle.unit_rms(kf, 1e-5) * kw.double()
    for i, s in enumerate(slots):
        blk, off = s // bs, s % bs
        assert (kc[blk, :, off].float().cpu().double().reshape(-1) - want_k[i]).abs().max().item() < tol * float(want_k.abs().max())
        assert torch.equal(vc[blk, :, off // 8, :, off % 8].cpu().reshape(-1), x[i, heads * dim:])


def test_mixing_head_weights_equals_mixing_crossed_outputs():
    """The definition - mix the heads' softmax weights by ``talk``, then apply head ``h``'s mixed weights to the values
    of the key / value head it belongs to - against what the framework computes: every head's weights on every value head, then
    ``mix_heads``."""
    from vllm_distributed_amd.ops import torch_ref
    g = torch.Generator().manual_seed(6)
    t, heads, kv, dim = 23, 6, 3, 8
    q, k = torch.randn(t, heads, dim, generator=g, dtype=F64), torch.randn(t, kv, dim, generator=g, dtype=F64)
    v = torch.randn(t, kv, dim, generator=g, dtype=F64)
    r1, r2 = torch.rand(heads, generator=g, dtype=F64), torch.rand(heads, generator=g, dtype=F64)
    talk = torch.randn(heads, heads, generator=g, dtype=F64)
    weights = oracle.softmax_weights(q, k, 0.3, r1, r2)
    mixed = torch.einsum("hg,gij->hij", talk, weights)
    want = torch.stack([mixed[h] @ v[:, h // 2] for h in range(heads)], 1).reshape(t, -1)
    crossed = torch.einsum("hij,jcd->ihcd", weights, v)                             # [T, H, kv, dim]
    got = torch_ref.mix_heads(crossed.float(), talk.float(), torch.float32).double()
    assert (got - want).abs().max().item() < 1e-5
    bs = 8
    table = torch.arange(3, dtype=torch.int32).view(1, -1)
    kc, vc = _paged(k.float(), v.float(), table, 3, bs, torch.float32)
    o = torch_ref.crossed_bias_attention(q.float(), kc, vc, table, torch.tensor([0, t]), torch.tensor([t]), 0.3,
                                         r1.float(), r2.float())
    assert (o.double() - crossed).abs().max().item() < 1e-5


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_convolution_tails_across_portions_first_tokens_and_stale_slots(device, dtype):
    """The input convolution (``x + conv(x)``, no activation) and the convolution with bias and SiLU, over a sequence
    cut into portions of many sizes: the tails come from the slot, the first tokens of a sequence read zeros whatever
    the slot's earlier owner left, and a second sequence in the same call does not disturb the first."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(8)
    c, n = 24, 61
    for taps in (1, 2, 4):
        x = torch.randn(n, c, generator=g).to(dt)
        other = torch.randn(5, c, generator=g).to(dt)
        wt = (torch.randn(c, taps, generator=g) * 0.5).to(dt)
        bias = torch.randn(c, generator=g)
        for silu, b, res in ((False, None, True), (True, bias, False)):
            y = oracle.causal_conv(x.double(), wt.double(), None if b is None else b.double())
            want = (oracle.silu(y) if silu else y) + (x.double() if res else 0.0)
            state = torch.full((3, max(taps - 1, 1), c), 9.0, dtype=dt, device=device)
            out, at, sizes = [], 0, [1, 1, 2, 3, 1, 17, 2, 30, 1, 1, 2]
            for i, m in enumerate(sizes):
                m = min(m, n - at)
                if i == 3:        # a stranger's portion rides along, in its own slot
                    rows = torch.cat([other, x[at:at + m]]).to(device)
                    got = ops.short_conv_act(rows, c, wt.t().contiguous().to(device), state, i32(device, 0, 1),
                                             i32(device, 0, 5, 5 + m), i32(device, 5, at + m),
                                             i32(device, *([0] * 5 + [1] * m)),
                                             i32(device, *(list(range(5)) + list(range(at, at + m)))), silu, True,
                                             None if b is None else b.to(device), res)[5:]
                else:
                    got = ops.short_conv_act(x[at:at + m].to(device), c, wt.t().contiguous().to(device), state,
                                             i32(device, 1), i32(device, 0, m), i32(device, at + m),
                                             None if m == 1 else i32(device, *([0] * m)),
                                             i32(device, *range(at, at + m)), silu, m > 1,
                                             None if b is None else b.to(device), res)
                out.append(got.float().cpu())
                at += m
            assert at == n
            got = torch.cat(out).double()
            assert (got - want).abs().max().item() < (2e-5 if dtype == "float32" else 0.06), (taps, silu)
            assert float(state[2].float().min()) == 9.0


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_gating_precedes_the_grouped_norm(device, dtype):
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(9)
    y, z = torch.randn(7, 48, generator=g) * 2, (torch.randn(7, 48, generator=g) * 2).to(dt)
    wgt = torch.rand(48, generator=g) + 0.5
    for parts in (1, 2, 6):
        got = ops.act_gate_group_norm(y.to(device), z.to(device), wgt.to(device), 1e-5, 48 // parts, dt).float().cpu().double()
        gated = y.double() * oracle.silu(z.double())
        want = oracle.unit_rms(gated.view(7, parts, -1), 1e-5).reshape(7, 48) * wgt.double()
        assert (got - want).abs().max().item() < (1e-5 if dtype == "float32" else 0.03)
        other = oracle.unit_rms(y.double().view(7, parts, -1), 1e-5).reshape(7, 48) * wgt.double() * oracle.silu(z.double())
        assert (got - other).abs().max().item() > 0.2                               # (norm first is another function)


@pytest.mark.parametrize("device", [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)])
def test_routing_rules(device):
    """The largest ``top`` sigmoid scores are chosen; the weights are those scores times the scale and nothing else
    (they do not sum to anything in particular)."""
    from vllm_distributed_amd.models.layers.moe import ScoredTopKMoE
    with torch.device(device):
        m = ScoredTopKMoE(32, 16, 6, 3, torch.float32, route_scale=1.5)
    g = torch.Generator().manual_seed(1)
    wr = torch.randn(6, 32, generator=g)
    m.gate.weight.data.copy_(wr)
    h = torch.randn(64, 32, generator=g)
    topw, topi = m.route(m.router_logits(h.to(device)))
    idx, wts = oracle.route(h.double(), {"r.router": wr}, "r.", 3, 1.5)
    assert torch.equal(topi.cpu().sort(-1).values, idx.sort(-1).values)
    assert (topw.cpu().gather(1, topi.cpu().argsort(-1)).double() - wts.gather(1, idx.argsort(-1))).abs().max().item() < 1e-6
    assert (topw.sum(-1) - 1).abs().max().item() > 0.5 and float(topw.max()) <= 1.5 and float(topw.min()) > 0


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
@pytest.mark.parametrize("hidden,ff,experts,top,shared", [(48, 24, 5, 2, 44), (128, 64, 4, 4, 0), (32, 16, 1, 1, 16)])
def test_expert_block_against_the_oracle(device, dtype, hidden, ff, experts, top, shared):
    from vllm_distributed_amd.models.layers.moe import ScoredTopKMoE
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(hidden)
    direction = torch.randn(hidden, generator=g) * 0.3
    w = {"m.router": (torch.arange(experts).float() - 1.0).view(-1, 1) * direction.view(1, -1)}
    for nm, f in [(f"e{e}", ff) for e in range(experts)] + ([("shared", shared)] if shared else []):
        w[f"m.{nm}.gate"] = torch.randn(f, hidden, generator=g) * hidden ** -0.5 * 1.5
        w[f"m.{nm}.up"] = torch.randn(f, hidden, generator=g) * hidden ** -0.5 * 1.5
        w[f"m.{nm}.down"] = torch.randn(hidden, f, generator=g) * f ** -0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    with torch.device(device):
        m = ScoredTopKMoE(hidden, ff, experts, top, dt, route_scale=1.3, shared_inter=shared)
    m.gate.weight.data.copy_(w["m.router"])
    for e in range(experts):
        for which, part in enumerate(("gate", "up")):
            m.w13.weight_loader(m.w13, w[f"m.e{e}.{part}"], (e, which))
        m.w2.weight_loader(m.w2, w[f"m.e{e}.down"], (e, 0))
    if shared:
        for which, part in enumerate(("gate", "up")):
            m.shared.w13.weight_loader(m.shared.w13, w[f"m.shared.{part}"], which)
        m.shared.w2.weight_loader(m.shared.w2, w["m.shared.down"])
    mlp = {"router": {"top": top, "scale": 1.3}, "shared": {"ff": shared} if shared else None}
    for rows in (1, 7, 200):
        h = (torch.randn(rows, hidden, generator=g) * 0.6).to(dt)
        routed, extra = m(h.to(device))
        assert (extra is None) == (shared == 0)
        got = routed.float().cpu().double() + (0.0 if extra is None else extra.float().cpu().double())
        want = oracle.moe_ff(h.double(), w, "m.", mlp)
        assert (got - want).abs().max().item() < (2e-5 if dtype == "float32" else 0.03) * max(1.0, want.abs().max().item())


def test_layers_caches_and_state(tmp_path_factory):
    """Every layer has the input convolution's tail as state; a recurrent layer adds its own convolution tail (model
    dtype) and its fp32 state; only attention layers own cache rows (key rows + values of equal size); nothing is
    windowed, so no page is given back while a request runs."""
    import types
    from vllm_distributed_amd.entrypoints import trace_replay
    path, cfg, w = model_dir("varied", tmp_path_factory)
    args = types.SimpleNamespace(model=path, dtype="bfloat16", out="", max_tokens=64, max_seqs=3, device="cpu",
                                 block_size=16, enforce_eager=True)
    core = trace_replay.make_core(args)
    try:
        mr = core.executor.driver.worker.model_runner
        model = mr.model
        owners = model.attention_layers()
        assert len(owners) == 2 and [a.layer_idx for a in owners] == [1, 3]
        assert tuple(owners[0].k_cache.shape[1:]) == (2, 16, 16) and tuple(owners[0].v_cache.shape[1:]) == (2, 2, 16, 8)
        states = model.state_layers()
        assert len(states) == 5 + 2 * 3 and len({id(s) for s in states}) == len(states)
        shapes = [tuple(s.shape) for s in mr.state_tensors]
        assert shapes[:3] == [(4, 2, 48), (4, 3, 4 * 12 + 2 * 2 * 10), (4, 4, 10, 12)]
        assert shapes[3] == (4, 2, 48) and shapes[4] == (4, 2, 48)
        assert shapes[5:7] == [(4, 3, 2 * 2 * 8 + 4 * 12), (4, 4, 8, 12)]
        dts = [s.dtype for s in mr.state_tensors]
        assert dts[:3] == [torch.bfloat16, torch.bfloat16, torch.float32] and dts[6] == torch.float32
        spec = mr.get_kv_cache_spec()
        assert spec.sliding_window is None
        assert spec.bytes_per_token == 2 * (2 * 2 * 16 + 2 * 3 * 8)
        names = [n for n, _ in model.named_parameters()]
        assert len(names) == len(set(names)) and "pos.weight" in names and not any("head" in n for n in names)
    finally:
        core.shutdown()


def test_config_errors():
    from vllm_distributed_amd.models.nalasun import NalasunLayer
    f32 = torch.float32
    ranks = {"l0.mix.a1": (4, 32), "l0.mix.g1": (4, 32)}
    NalasunLayer(32, delta(2, 1, 8, 8, 3, moe(3, 2, 8)), 1e-5, 3, 0, f32, ranks)
    with pytest.raises(ValueError):                                               # no tensor states the ranks
        NalasunLayer(32, delta(2, 1, 8, 8, 3), 1e-5, 3, 0, f32, {})
    stated = delta(2, 1, 8, 8, 3)
    stated["mixer"].update(decay_rank=4, gate_rank=4)
    NalasunLayer(32, stated, 1e-5, 3, 0, f32, {})
    for bad in (attention(4, 3, 8, 0.2), dict(attention(2, 1, 8, 0.2), type="other"), delta(3, 2, 8, 8, 3),
                ssm(4, 8, 4, 3, 1, 2), ssm(3, 8, 4, 1, 5, 2), ssm(2, 8, 4, 1, 1, 2, dict(moe(3, 2, 8), kind="other")),
                attention(2, 1, 8, 0.2, None, moe(3, 4, 8))):
        with pytest.raises(ValueError):
            NalasunLayer(32, bad, 1e-5, 3, 0, f32, ranks)
    wrong = attention(2, 1, 8, 0.2)
    wrong["mixer"]["vdim"] = 16                                                   # the values are the keys
    with pytest.raises(ValueError):
        NalasunLayer(32, wrong, 1e-5, 3, 0, f32, ranks)


def test_dummy_weights_and_config_keys():
    """Random-weight loading (the benchmark's path): every parameter is filled, the derived keys are there."""
    from vllm_distributed_amd.config import normalize_hf_config
    from vllm_distributed_amd.models.nalasun import weight_shapes
    cfg = json.loads(json.dumps(CONFIGS["paged"]))
    for spec in cfg["layers"]:
        if spec["type"] == "channel_delta":
            spec["mixer"].update(decay_rank=5, gate_rank=7)
    shapes = weight_shapes(cfg)
    assert shapes["l1.mix.a2"] == (4 * 16, 5) and shapes["l1.mix.g1"] == (7, 64) and shapes["l0.canon1"] == (64, 4)
    assert shapes["l2.mix.in"] == (2 * 64 + 2 * 2 * 16 + 4, 64) and shapes["l2.mix.conv.b"] == (64 + 64,)
    assert shapes["l0.mlp.shared.down"] == (64, 32) and "l1.mlp.shared.up" not in shapes and "l3.norm2" not in shapes
    assert shapes["l0.mix.talk"] == (4, 4) and shapes["pos"] == (400, 64) and "head" not in shapes
    n = dict(cfg)
    normalize_hf_config(n)
    assert n["hidden_size"] == 64 and n["vocab_size"] == 97 and n["num_hidden_layers"] == 4
    assert n["max_position_embeddings"] == 400 and n["architectures"] == ["NalasunForCausalLM"]
    from vllm_distributed_amd import LLM, SamplingParams
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(cfg, f)
        llm = LLM(model=d, device="cpu", dtype="float32", max_model_len=64, max_num_seqs=2, block_size=16,
                  load_format="dummy", enforce_eager=True)
        try:
            out = llm.generate([[1, 2, 3]], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
        finally:
            llm.shutdown()
        assert len(out[0].outputs[0].token_ids) == 4


def test_sizes_that_only_tensor_shapes_state(tmp_path_factory, tmp_path):
    """A config that leaves out what the tensors' shapes say anyway - the taps of every convolution, the low-rank
    widths, the number of positions - loads and computes the same model."""
    from safetensors.torch import save_file
    path, cfg, w = model_dir("paged", tmp_path_factory)
    bare = json.loads(json.dumps(cfg))
    bare.pop("canon")
    bare.pop("max_positions")
    for spec in bare["layers"]:
        spec["mixer"].pop("conv", None)
    d = tmp_path / "bare"
    d.mkdir()
    save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    (d / "config.json").write_text(json.dumps(bare))
    toks = tokens_for(cfg, 40, 70)
    got = run_schedule(str(d), portions(toks, [17, 1], "r"), "float32", "cpu", max_tokens=64, tmp=tmp_path)
    check(got, "paged", cfg, w, {"r": toks}, 2e-4)


def test_the_trace_runner_as_a_program(tmp_path_factory, tmp_path):
    import subprocess
    import sys
    path, cfg, w = model_dir("degenerate", tmp_path_factory)
    a, b = tokens_for(cfg, 9, 50), tokens_for(cfg, 5, 51)
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": []}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[6:], "want": [2]}], "end": ["a"]}]
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    r = subprocess.run([sys.executable, exe, "--model", path, "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "128",
                        "--device", "cpu"], input="".join(json.dumps(x) + "\n" for x in lines), text=True,
                       capture_output=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = oracle_logits("degenerate", cfg, w, a)
    got0 = np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, cfg["vocab"])
    got2 = np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, cfg["vocab"])
    assert np.abs(got0 - want[[0, 5]]).max() < 2e-4 and np.abs(got2 - want[[8]]).max() < 2e-4


# ------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_greedy_generation_through_the_scheduler(device, dtype, tmp_path_factory):
    """``LLM.generate`` on five prompts with two sequence slots and small prefill chunks: the scheduler's own batching,
    chunking and sampling.  Every generated token is the oracle's argmax given the tokens before it (in bfloat16: or
    its logit is within rounding of the oracle's best)."""
    from vllm_distributed_amd import LLM, SamplingParams
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (3, 30, 1, 17, 45)]
    llm = LLM(model=path, device=device, dtype=dtype, max_model_len=128, max_num_seqs=2, max_num_batched_tokens=16,
              block_size=16, load_format="safetensors", enforce_eager=False)
    try:
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    finally:
        llm.shutdown()
    for prompt, o in zip(prompts, outs):
        gen = list(o.outputs[0].token_ids)
        assert len(gen) == 24
        logits = oracle.forward(cfg, w, prompt + gen).numpy()
        for i, tok in enumerate(gen):
            row = logits[len(prompt) + i - 1]
            if dtype == "float32":
                assert tok == int(row.argmax()), (len(prompt), i)
            else:
                assert row.max() - row[tok] < 0.3, (len(prompt), i, float(row.max() - row[tok]))
                if row.max() - row[tok] > 0:              # a near-tie went the other way: later tokens follow another text
                    break
