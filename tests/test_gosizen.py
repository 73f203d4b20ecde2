"""Gosizen through the framework (loader, scheduler, block and state-slot bookkeeping, model runner, kernels on the
GPU / reference ops on the CPU) against the plain float64 model of ``tests/gosizen_oracle.py``.

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

import gosizen_oracle as oracle
from test_tavulix import portions, run_schedule, tokens_for

F64 = torch.float64


# ------------------------------------------------------------------------------------------------ models
def latent(heads, dim, rot_dim, vdim, rank, q_rank, window, mlp=None, base=10000.0, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank,
         "scale": scale or (dim + rot_dim) ** -0.5, "mask": {"size": window},
         "rot": {"base": base, "dims": rot_dim}}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def left(heads, kv, dim, vdim, conv, chunk, rot_dims, scaling=True, base=5000.0, scale=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 48}
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale or dim ** -0.5,
            "mask": {"size": chunk}, "rot": rot}


def right(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def parallel(l, r, ls, rs, mlp=None):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(layers, width=48, vocab=97, eps=1e-5, loop=None, side=8, cap=12.0):
    c = {"architecture": "Gosizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if side:
        c["token_side"] = {"dim": side}
    if cap:
        c["logit_softcap"] = cap
    return c


# (the widths of the two low-rank projections of a right half are sizes only the tensors state)
RANKS = {"varied": (6, 10), "degenerate": (3, 3), "paged": (5, 7), "plain": (4, 4), "wide": (8, 8), "uneven": (5, 9)}

CONFIGS = {
    # every layer of another shape; a loop over a latent and a parallel layer run three times; a parallel layer in
    # front of the loop; partial rotation; several value heads per query / key head on the right; a layer without
    # feed-forward; windows and chunks of a few tokens
    "varied": config([
        parallel(left(4, 2, 16, 8, 3, 7, 8), right(4, 2, 8, 12, 4), 0.7, 0.4, moe(5, 2, 24)),
        latent(3, 12, 8, 20, 24, 20, 9, dense(64)),
        parallel(left(6, 3, 8, 16, 2, 5, 8, scaling=False), right(2, 2, 16, 8, 3), 1.1, 0.9, None),
        latent(2, 8, 4, 8, 12, 16, 4, moe(4, 3, 16))], loop=(1, 3, 3)),
    # values a model can make equal or one: one head, kv heads = heads, vdim = dim, one tap, a window and a chunk of
    # one token and ones wider than any test sequence, top 1 of 1 expert and top = experts, a loop that runs once, a
    # loop that starts at layer 0 and covers every layer, scales of exactly one, no side input, no logit cap
    "degenerate": config([
        latent(1, 16, 16, 16, 16, 8, 1, moe(1, 1, 16), base=100.0),
        parallel(left(2, 2, 8, 8, 1, 1, 8, scaling=False), right(1, 1, 8, 8, 1), 1.0, 1.0, moe(3, 3, 8)),
        parallel(left(1, 1, 16, 16, 4, 400, 4), right(2, 2, 8, 8, 2), 1.0, 1.0, dense(32)),
        latent(2, 8, 2, 8, 8, 8, 400, None)], width=32, vocab=50, loop=(0, 4, 1), side=0, cap=0.0),
    # windows and chunks that span pages of 16 tokens; the loop is the tail of the model
    "paged": config([
        latent(4, 16, 8, 16, 32, 24, 37, dense(96)),
        parallel(left(4, 1, 32, 16, 3, 40, 16), right(4, 2, 16, 16, 4), 0.6, 0.5, moe(6, 2, 32)),
        latent(2, 16, 8, 8, 16, 16, 21, moe(4, 2, 32))], width=64, loop=(1, 3, 2), side=4),
    # no loop at all
    "plain": config([parallel(left(2, 1, 16, 8, 3, 11, 16), right(2, 1, 8, 8, 4), 0.5, 0.5, dense(48)),
                     latent(2, 8, 8, 8, 16, 16, 6, dense(48))], width=32, side=6),
    # sizes the 16-bit kernels' 16-byte and matrix-core paths take (head sizes of 32 / 64, a rotated half of 16, latent
    # rows of 64 + 32 values)
    "wide": config([parallel(left(4, 2, 64, 32, 3, 24, 32), right(4, 4, 32, 32, 4), 0.6, 0.5, moe(4, 2, 64)),
                    latent(4, 32, 32, 32, 64, 64, 20, dense(128))], width=128, loop=(0, 2, 2), side=8),
    # a width, a vocabulary and sizes that are no multiples of 8 (no 16-byte access fits a 16-bit row)
    "uneven": config([
        latent(3, 10, 6, 14, 22, 18, 30, moe(5, 2, 30), base=3000.0),
        parallel(left(3, 1, 20, 12, 3, 45, 10), right(3, 3, 12, 20, 4), 0.8, 0.3, dense(50)),
        parallel(left(2, 2, 12, 12, 4, 64, 12), right(4, 1, 20, 10, 2), 0.5, 0.7, moe(3, 1, 26))],
        width=100, vocab=211, loop=(1, 3, 2), side=6, cap=9.0),
}


def random_weights(cfg, seed, ranks):
    g = torch.Generator().manual_seed(seed)
    width, n = cfg["width"], len(cfg["layers"])

    def rnd(*shape, lo=-1.0, hi=1.0):
        return lo + (hi - lo) * torch.rand(shape, generator=g)

    def proj(rows, cols, gain=1.0):
        return rnd(rows, cols) * gain * (3.0 / cols) ** 0.5

    w = {"embed": rnd(cfg["vocab"], width), "head": proj(cfg["vocab"], width), "final.norm": rnd(width, lo=-0.3, hi=0.4)}
    side = (cfg.get("token_side") or {}).get("dim")
    if side:
        w["side.embed"] = rnd(cfg["vocab"], side * n)
    if cfg.get("loop"):
        w["loop.in"], w["loop.step"] = proj(width, 2 * width, 1.4), rnd(cfg["loop"]["times"], width, lo=-0.5, hi=0.5)
    for i, spec in enumerate(cfg["layers"]):
        m, p = spec["mixer"], f"l{i}."
        w[p + "norm1"] = rnd(width, lo=-0.3, hi=0.4)
        if spec["type"] == "latent_attention":
            heads, q = m["heads"], p + "mix."
            # (scores of a few units: a softmax that is nearly one-hot multiplies every rounding step before it)
            w[q + "dq"], w[q + "dq.norm"] = proj(m["q_rank"], width), rnd(m["q_rank"], lo=0.6, hi=1.4)
            w[q + "uq"] = proj(heads * (m["dim"] + m["rot_dim"]), m["q_rank"], 1.5)
            w[q + "dkv"], w[q + "dkv.norm"] = proj(m["kv_rank"] + m["rot_dim"], width), rnd(m["kv_rank"], lo=0.6, hi=1.4)
            w[q + "uk"], w[q + "uv"] = proj(heads * m["dim"], m["kv_rank"]), proj(heads * m["vdim"], m["kv_rank"])
            w[q + "sink"], w[q + "g"] = rnd(heads, lo=-1.0, hi=2.0), proj(heads, width, 2.0)
            w[q + "o"] = proj(width, heads * m["vdim"])
        else:
            l, q = m["left"], p + "mix.left."
            for nm, rows in (("q", l["heads"] * l["dim"]), ("k", l["kv_heads"] * l["dim"]), ("v", l["kv_heads"] * l["vdim"])):
                w[q + nm], w[q + nm + ".b"], w[q + nm + ".conv"] = proj(rows, width), rnd(rows, lo=-0.3, hi=0.3), rnd(rows, l["conv"], lo=-0.7, hi=0.7)
            w[q + "sink"], w[q + "g"] = rnd(l["heads"], lo=-1.0, hi=2.0), proj(l["heads"] * l["vdim"], width, 2.0)
            w[q + "o"] = proj(width, l["heads"] * l["vdim"])
            r, q = m["right"], p + "mix.right."
            for nm, rows in (("q", r["kv_heads"] * r["dim"]), ("k", r["kv_heads"] * r["dim"]), ("v", r["heads"] * r["vdim"])):
                w[q + nm], w[q + nm + ".conv"] = proj(rows, width, 2.0), rnd(rows, r["conv"])
            w[q + "b"], w[q + "A_log"], w[q + "norm"] = proj(r["heads"], width, 2.0), rnd(r["heads"], lo=-2.5, hi=0.5), rnd(r["vdim"], lo=0.6, hi=1.4)
            w[q + "a1"], w[q + "a2"] = proj(ranks[0], width, 2.0), proj(r["heads"] * r["dim"], ranks[0], 2.0)
            w[q + "dt_bias"] = rnd(r["heads"] * r["dim"], lo=-1.0, hi=1.0)
            w[q + "g1"], w[q + "g2"] = proj(ranks[1], width, 2.0), proj(r["heads"] * r["vdim"], ranks[1], 2.0)
            w[q + "o"] = proj(width, r["heads"] * r["vdim"])
        mlp = spec["mlp"]
        if mlp and mlp["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = proj(mlp["ff"], width, 1.5), proj(width, mlp["ff"])
        elif mlp:
            for e in range(mlp["router"]["experts"]):
                w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = proj(mlp["expert"]["ff"], width, 2.0), proj(width, mlp["expert"]["ff"])
            w[p + "mlp.router"], w[p + "mlp.router.b"] = proj(mlp["router"]["experts"], width, 3.0), rnd(mlp["router"]["experts"], lo=-0.5, hi=0.5)
        if side:
            w[p + "side.gate"], w[p + "side.proj"], w[p + "side.norm"] = proj(side, width, 2.0), proj(width, side), rnd(width, lo=0.3, hi=0.9)
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


_MODELS = {}


def model_dir(name, tmp_path_factory, dtype="float32"):
    """The model's folder, configuration and weights.  For bfloat16 runs the routers are made decisive: their weights
    are made small and their biases set 1.5 apart in a random order, so that every token chooses the same experts
    whatever rounding does to the logits - the weights of the chosen still differ from token to token.  In bfloat16 the router's input carries the
    rounding of every layer before it, and a close call that falls the other way swaps a whole expert; the float32
    runs keep the free-running routers."""
    decisive = dtype != "float32"
    if (name, decisive) not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]
        w = random_weights(cfg, sum(map(ord, name)), RANKS[name])
        if decisive:
            g = torch.Generator().manual_seed(11)
            for k in [k for k in w if k.endswith(".router.b")]:
                w[k] = (torch.randperm(w[k].numel(), generator=g) * 1.5 - w[k].numel()).to(torch.bfloat16)
                w[k[:-2]] = (w[k[:-2]].float() * 0.05).to(torch.bfloat16)
        d = tmp_path_factory.mktemp("gosizen_" + name)
        save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[(name, decisive)] = (str(d), cfg, w)
    return _MODELS[(name, decisive)]


_ORACLE = {}


def oracle_logits(name, cfg, w, tokens):
    key = (name, id(w), tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = oracle.forward(cfg, w, list(tokens)).numpy()
    return _ORACLE[key]


def check(got, name, cfg, w, reqs, tol):
    """Every row the run produced against the oracle.  A few rows in a hundred may lie outside the tolerance, by a
    factor of three at most: the recurrent layer's output is normed per head, so at a position where that output nearly
    cancels, the rounding of its inputs is multiplied up (the reference ops show the same rows, in float32 fifty times
    further off than their neighbours); a wrong index or a lost state shows in many rows, and by far more."""
    assert got
    errs = sorted(((float(np.abs(row - oracle_logits(name, cfg, w, reqs[rid])[p]).max()), rid, p)
                   for (rid, p), row in got.items()), reverse=True)
    allowed = max(1, len(errs) // 50)
    assert errs[0][0] <= 3 * tol, errs[0]
    assert errs[allowed][0] <= tol if len(errs) > allowed else True, errs[:allowed + 1]


DEVICES = [pytest.param("cpu", "float32", 2e-4, id="cpu-f32"),
           pytest.param("cuda", "float32", 2e-4, id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", 0.35, id="gpu-bf16", marks=pytest.mark.gpu)]


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
def test_residual_stream_after_every_layer_run(device, dtype, tol, tmp_path_factory):
    """The fp32 residual stream after every run of a layer (a looped layer counts each time)."""
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
    assert len(got) == len(want) == 1 + 2 * 3 + 1
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item()), i


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", ["varied", "paged", "wide"])
def test_prefill_then_long_token_by_token_decoding(name, device, dtype, tol, tmp_path_factory, tmp_path):
    """A prompt, then 150 tokens one at a time: state and convolution tails are carried through 150 single-row steps,
    every window and chunk passes over decoded tokens, the cache grows over several pages while the pages behind the
    widest window go back to the pool."""
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    toks = tokens_for(cfg, 190, 4)
    got = run_schedule(path, portions(toks, [40, 1], "r"), dtype, device, max_tokens=192, tmp=tmp_path)
    assert len(got) == 190
    check(got, name, cfg, w, {"r": toks}, tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 0.35)])
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
    """Portions cut inside windows, chunks and pages, down to two tokens and one."""
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
def test_the_delta_rule_overwrites_and_forgets_and_stale_slots_do_not_show(device, dtype):
    """Token 0 writes value A under a key, token 150 writes value B under the same key with beta ~ 1: a query for the
    key at the end returns B, not A + B (the delta rule takes the old value out); a head whose decay forgets returns
    nothing of a far write.  The sequence runs in portions of many sizes through a slot another sequence left full,
    and the whole is compared with the token-by-token float64 recurrence."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    heads, qk, dim, vdim, n = 2, 1, 8, 8, 301
    g = torch.Generator().manual_seed(3)
    q = torch.randn(n, qk, dim, generator=g) * 0.02
    k = torch.randn(n, qk, dim, generator=g) * 0.02
    v = torch.randn(n, heads, vdim, generator=g) * 0.05
    k[0, 0, 0], k[150, 0, 0], q[n - 1, 0, 0] = 5.0, 5.0, 5.0
    v[0, :, 1], v[150, :, 2] = 4.0, 3.0
    beta = torch.full((n, heads), -14.0)          # (q and k become unit vectors: the other tokens must not write)
    beta[0], beta[150] = 9.0, 9.0
    x = torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], 1).to(dt)
    beta, dtr = beta.to(dt), torch.zeros(n, heads * dim).to(dt)
    # head 0 keeps (decay ~ 0.9995 per token), head 1 forgets (~ 0.5)
    a_log = torch.tensor([math.log(0.0005 / math.log(2.0)), 0.0])
    dt_bias = torch.zeros(heads * dim)
    xf = x.double()
    qn = xf[:, :dim].view(n, qk, dim)
    kn = xf[:, dim:2 * dim].view(n, qk, dim)
    qn = (qn / torch.sqrt((qn * qn).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5).repeat_interleave(heads, 1)
    kn = (kn / torch.sqrt((kn * kn).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(heads, 1)
    decay = torch.exp(-torch.exp(a_log.double()).view(1, heads, 1) * math.log(2.0)).expand(n, heads, dim)
    want, _ = oracle.delta_heads(qn, kn, xf[:, 2 * dim:].view(n, heads, vdim), oracle.sigmoid(beta.double()), decay)
    last = want[n - 1, 0] * dim ** 0.5
    assert abs(float(last[2]) - 3.0 * 0.9995 ** 150) < 0.1 and abs(float(last[1])) < 0.1       # B alone, A taken out
    assert want[n - 1, 1].abs().max().item() < 0.05                                           # the forgetting head
    state = torch.full((3, heads, dim, vdim), 7.0, device=device)                  # what an earlier owner left
    out, at, sizes = [], 0, [1, 2, 64, 17, 1, 1, 100, 3, 2]
    for i in range(100):
        m = min(sizes[i % len(sizes)], n - at)
        if m == 0:
            break
        out.append(ops.gated_delta_rule(x[at:at + m].to(device), heads, qk, dim, vdim, beta[at:at + m].to(device),
                                        dtr[at:at + m].to(device), dt_bias.to(device), a_log.to(device), state,
                                        i32(device, 2), i32(device, 0, m), i32(device, at + m)).cpu())
        at += m
    got = torch.cat(out).view(n, heads, vdim).double()
    assert (got - want).abs().max().item() < (2e-4 if dtype == "float32" else 2e-3)


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
@pytest.mark.parametrize("dim,vdim,heads,qk", [(24, 20, 3, 1), (32, 32, 4, 4), (96, 40, 2, 2), (160, 16, 1, 1), (10, 7, 2, 2), (66, 33, 2, 1)])
def test_delta_rule_sizes(device, dtype, dim, vdim, heads, qk):
    """Head sizes on both sides of every tiling of the recurrence kernel, value heads sharing query / key heads, two
    sequences in one call (one continuing from a state, one starting)."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(dim)
    n = [9, 5]
    t = sum(n)
    x = (torch.randn(t, 2 * qk * dim + heads * vdim, generator=g) * 0.7).to(dt)
    beta = torch.randn(t, heads, generator=g).to(dt)
    dtr = torch.randn(t, heads * dim, generator=g).to(dt)
    dt_bias, a_log = torch.randn(heads * dim, generator=g) * 0.5, torch.randn(heads, generator=g) - 1.0
    s0 = torch.randn(heads, dim, vdim, generator=g) * 0.3
    state = torch.full((4, heads, dim, vdim), 5.0)
    state[1] = s0
    state = state.to(device)
    got = ops.gated_delta_rule(x.to(device), heads, qk, dim, vdim, beta.to(device), dtr.to(device), dt_bias.to(device),
                               a_log.to(device), state, i32(device, 1, 3), i32(device, 0, n[0], t),
                               i32(device, 20 + n[0], n[1])).cpu().double().view(t, heads, vdim)
    xf = x.double()
    qn, kn = xf[:, :qk * dim].view(t, qk, dim), xf[:, qk * dim:2 * qk * dim].view(t, qk, dim)
    qn = (qn / torch.sqrt((qn * qn).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5).repeat_interleave(heads // qk, 1)
    kn = (kn / torch.sqrt((kn * kn).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(heads // qk, 1)
    decay = torch.exp(-torch.exp(a_log.double()).view(1, heads, 1)
                      * oracle.softplus(dtr.double().view(t, heads, dim) + dt_bias.double().view(1, heads, dim)))
    v, b = xf[:, 2 * qk * dim:].view(t, heads, vdim), oracle.sigmoid(beta.double())
    w0, e0 = oracle.delta_heads(qn[:n[0]], kn[:n[0]], v[:n[0]], b[:n[0]], decay[:n[0]], s0.double())
    w1, e1 = oracle.delta_heads(qn[n[0]:], kn[n[0]:], v[n[0]:], b[n[0]:], decay[n[0]:])
    tol = 2e-4 if dtype == "float32" else 2e-3
    assert (got - torch.cat([w0, w1])).abs().max().item() < tol
    assert (state[1].cpu().double() - e0).abs().max().item() < tol and (state[3].cpu().double() - e1).abs().max().item() < tol
    assert float(state[0].min()) == 5.0 and float(state[2].max()) == 5.0


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_one_key_stands_out_at_window_edges_and_page_borders(device, dtype):
    """Latent rows in shuffled pages of 16 and a window of 40; the query is aimed at ONE key: the output is that row's
    latent part exactly when the key is the row itself or one of the 39 before it - the last one inside, the first one
    outside, across page borders, for a decoded row and a prompt's row; the sink takes its share; the gate scales.
    Pages wholly behind the window are poisoned: they are never read."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    n, rank, rope, bs, heads, window = 330, 16, 8, 16, 2, 40
    g = torch.Generator().manual_seed(9)
    nblk = -(-n // bs) + 2
    table = torch.randperm(nblk, generator=g)[:-(-n // bs)].to(torch.int32).view(1, -1)
    rows = torch.randn(n, rank + rope, generator=g) * 0.3
    cache = torch.zeros(nblk, 1, bs, rank + rope)
    for j in range(n):
        cache[table[0, j // bs], 0, j % bs] = rows[j]
    cache = cache.to(dt)
    stored = cache.float()
    for pos in (329, 300, 47, 40, 39, 17, 0):
        poisoned = cache.clone()
        for blk in range((pos + 1 - window) // bs if pos + 1 >= window else 0):
            poisoned[table[0, blk]] = float("nan")
        dev_cache, dev_table = poisoned.to(device), table.clone()
        dev_table[0, :max((pos + 1 - window) // bs, 0)] = nblk - 1                # released pages may name anything
        dev_table = dev_table.to(device)
        for target in sorted({pos, pos - 1, pos - 38, pos - 39, pos - 40, pos - 41, pos // bs * bs, pos // bs * bs - 1}):
            if target < 0:
                continue
            key = stored[table[0, target // bs], 0, target % bs]
            q = (key * 60 / key.norm() ** 2).view(1, 1, -1).repeat(1, heads, 1).to(dt).to(device)
            seen = pos - target < window
            for token_seq in (None, i32(device, 0)):                               # a decoded row / a prompt's row
                o = ops.latent_row_attention(q, dev_cache, dev_table, token_seq, i32(device, pos + 1), 1.0, rank, 0, window)
                assert not torch.isnan(o).any(), (pos, target)
                hit = (o[0, 0].float().cpu() - key[:rank]).abs().max().item() < 0.05
                assert hit == seen, (target, pos)
    # sink and gate in closed form: one visible key with score s, sink k -> weight e^s / (e^s + e^k), times sigmoid(g)
    key = stored[table[0, 0], 0, 0]
    q = (key * 2.0 / key.norm() ** 2).view(1, 1, -1).repeat(1, heads, 1).to(dt).to(device)
    s = float((q[0, 0].float().cpu() * key).sum())
    sinks, gate = torch.tensor([1.5, -0.5]), torch.tensor([[0.3, -1.2]])
    o = ops.latent_row_attention(q, cache.to(device), table.to(device), None, i32(device, 1), 1.0, rank, 0, window,
                                 sinks.to(device), gate.to(dt).to(device)).float().cpu()
    for h in range(heads):
        wgt = math.exp(s) / (math.exp(s) + math.exp(float(sinks[h]))) / (1 + math.exp(-float(gate.to(dt).float()[0, h])))
        assert (o[0, h] - key[:rank] * wgt).abs().max().item() < (1e-5 if dtype == "float32" else 5e-3)


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
@pytest.mark.parametrize("dim,vdim", [(8, 8), (32, 16)])
def test_one_key_stands_out_at_chunk_edges(device, dtype, dim, vdim):
    """Key rows and values in shuffled pages of 16 and chunks of 24 positions counted from the sequence's start; the
    query is aimed at ONE key: it is seen exactly when it lies in the query's own chunk at or before it - the chunk's
    first key, the last key of the chunk before, across page borders; as a decoded row and as the last row of a prompt
    portion that starts in the chunk before."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    n, bs, chunk, hq, hkv = 130, 16, 24, 2, 1
    g = torch.Generator().manual_seed(dim)
    nblk = -(-n // bs) + 1
    table = torch.randperm(nblk, generator=g)[:-(-n // bs)].to(torch.int32).view(1, -1)
    keys = torch.randn(n, dim, generator=g) * 0.3
    vals = torch.randn(n, vdim, generator=g)
    kc, vc = torch.zeros(nblk, hkv, bs, dim), torch.zeros(nblk, hkv, bs // 8, vdim, 8)
    for j in range(n):
        b, off = int(table[0, j // bs]), j % bs
        kc[b, 0, off], vc[b, 0, off // 8, :, off % 8] = keys[j], vals[j]
    kc, vc = kc.to(dt), vc.to(dt)
    aim = torch.zeros(dim)
    aim[1] = 3.0                                           # the target's key: far longer than any other key
    for pos in (129, 120, 119, 96, 95, 48, 47, 24, 23, 0):
        lo = pos // chunk * chunk
        for target in sorted({pos, lo, lo - 1, lo + 1, pos - 1, lo - chunk, max(pos // bs * bs - 1, 0)}):
            if target < 0 or target > pos:
                continue
            kt = kc.clone()
            kt[table[0, target // bs], 0, target % bs] = aim.to(dt)
            kt, vd = kt.to(device), vc.to(device)
            seen = target >= lo
            for rows in (1, min(9, pos + 1)):
                q = torch.randn(rows, hq, dim, generator=g) * 0.01
                q[-1] = aim * 20 / 3.0
                q = q.to(dt).to(device)
                positions = torch.arange(pos - rows + 1, pos + 1, dtype=torch.int32, device=device)
                o = ops.window_bias_attention(q, kt, vd, table.to(device), i32(device, 0, rows), i32(device, pos + 1),
                                              None if rows == 1 else torch.zeros(rows, dtype=torch.int32, device=device),
                                              positions, 1.0, 0.0, chunk, 0, None, None, None, None, rows, chunk=chunk)
                want = vc[table[0, target // bs], 0, (target % bs) // 8, :, target % 8].float()
                hit = (o[-1, 0].float().cpu() - want).abs().max().item() < 0.05
                assert hit == seen, (target, pos, rows)


@pytest.mark.parametrize("device", [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)])
def test_routing_rules(device):
    """The largest ``top`` of logits + bias, weights = softmax over the chosen only (they sum to one); a bias can
    carry an expert into every choice."""
    from vllm_distributed_amd.models.layers.moe import BiasedTopKMoE
    with torch.device(device):
        m = BiasedTopKMoE(32, 16, 6, 3, torch.float32)
    g = torch.Generator().manual_seed(1)
    wr, b = torch.randn(6, 32, generator=g), torch.tensor([0.0, 0.3, -0.2, 50.0, 0.1, -0.4])
    m.gate.weight.data.copy_(wr)
    m.gate_bias.data.copy_(b)
    h = torch.randn(64, 32, generator=g)
    topw, topi = m.route(m.router_logits(h.to(device)))
    idx, wts = oracle.route(h.double(), {"r.router": wr, "r.router.b": b}, "r.", 3)
    assert torch.equal(topi.cpu().sort(-1).values, idx.sort(-1).values)
    assert (topw.cpu().gather(1, topi.cpu().argsort(-1)).double() - wts.gather(1, idx.argsort(-1))).abs().max().item() < 1e-6
    assert (topw.sum(-1) - 1).abs().max().item() < 1e-5 and (topi == 3).any(-1).all()


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
@pytest.mark.parametrize("hidden,ff,experts,top", [(48, 24, 5, 2), (128, 64, 4, 4), (32, 16, 1, 1)])
def test_expert_block_against_the_oracle(device, dtype, hidden, ff, experts, top):
    from vllm_distributed_amd.models.layers.moe import BiasedTopKMoE
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(hidden)
    w = {"m.router": torch.randn(experts, hidden, generator=g) * 0.5, "m.router.b": torch.arange(experts) * 3.0}
    for e in range(experts):
        w[f"m.e{e}.up"] = torch.randn(ff, hidden, generator=g) * hidden ** -0.5 * 1.5
        w[f"m.e{e}.down"] = torch.randn(hidden, ff, generator=g) * ff ** -0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    with torch.device(device):
        m = BiasedTopKMoE(hidden, ff, experts, top, dt)
    m.gate.weight.data.copy_(w["m.router"])
    m.gate_bias.data.copy_(w["m.router.b"].float())
    for e in range(experts):
        m.w1.weight_loader(m.w1, w[f"m.e{e}.up"], e)
        m.w2.weight_loader(m.w2, w[f"m.e{e}.down"], e)
    for rows in (1, 7, 200):
        h = (torch.randn(rows, hidden, generator=g) * 0.6).to(dt)
        got = m(h.to(device)).float().cpu().double()
        want = oracle.moe_ff(h.double(), w, "m.", {"router": {"top": top}})
        assert (got - want).abs().max().item() < (2e-5 if dtype == "float32" else 0.03) * max(1.0, want.abs().max().item())


def test_rotations_and_frequencies():
    """Both pairings against a rotation written pair by pair, partial rotation, and the wavelength bands of the
    frequency scaling: short wavelengths kept, long ones slowed by the factor, the band between blended."""
    from vllm_distributed_amd.models.layers.attention import rotary_frequencies
    from vllm_distributed_amd.ops import torch_ref
    rot = {"base": 300.0, "dims": 12, "scaling": {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 40}}
    f, mult = rotary_frequencies(12, 300.0, rot["scaling"])
    want = oracle.frequencies(rot)
    assert mult == 1.0 and (f.double() - want).abs().max().item() < 1e-7
    plain = torch.tensor([300.0 ** (-2 * i / 12) for i in range(6)], dtype=F64)
    lam = 2 * math.pi / plain
    assert any(l < 40 / 3 for l in lam) and any(l > 40 for l in lam) and any(40 / 3 <= l <= 40 for l in lam)
    for i in range(6):
        if lam[i] < 40 / 3:
            assert abs(float(want[i] - plain[i])) < 1e-12
        elif lam[i] > 40:
            assert abs(float(want[i] - plain[i] / 5)) < 1e-12
        else:
            assert plain[i] / 5 < want[i] < plain[i]
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 3, 16, generator=g)
    pos = torch.tensor([0, 1, 7, 300, 4000])
    for inter in (False, True):
        got = torch_ref.rotate_pairs_first(x, pos, f, 1.0, inter).double()
        assert (got - oracle.rotate(x.double(), pos, rot, inter)).abs().max().item() < 2e-4
        assert torch.equal(got[..., 12:], x[..., 12:].double()) and torch.equal(got[0], x[0].double())


def test_norms_side_input_and_activations_against_the_oracle():
    from vllm_distributed_amd.ops import torch_ref
    g = torch.Generator().manual_seed(5)
    x, a, b, y = (torch.randn(7, 24, generator=g) for _ in range(4))
    w, pw = torch.randn(24, generator=g) * 0.2, torch.rand(24, generator=g)
    res = x.clone()
    out = torch_ref.add_rms_norm_to(res, a, b, w, 1e-5, torch.float32, 1.0)
    assert (res.double() - (x + a + b).double()).abs().max().item() < 1e-6
    assert (out.double() - oracle.offset_norm((x + a + b).double(), w, 1e-5)).abs().max().item() < 1e-5
    res2 = x.clone()
    out2 = torch_ref.norm_add_norm(y, pw, res2, w, 1e-5, torch.float32, 1.0)
    want = x.double() + oracle.unit_rms(y.double(), 1e-5) * pw.double()
    assert (res2.double() - want).abs().max().item() < 1e-5
    assert (out2.double() - oracle.offset_norm(want, w, 1e-5)).abs().max().item() < 1e-5
    z = torch.linspace(-6, 6, 97)
    assert (torch_ref.gelu_tanh_f(z).double() - oracle.gelu_tanh(z.double())).abs().max().item() < 1e-6
    assert (oracle.gelu_tanh(z.double()) - oracle.gelu_erf(z.double())).abs().max().item() > 1e-4      # two different curves
    table, ids = torch.randn(11, 12, generator=g), torch.tensor([3, 0, 10, 3, 7, 1, 1], dtype=torch.int32)
    gate = torch.randn(7, 4, generator=g)
    got = torch_ref.gelu_mul_rows(gate, table, ids, 8)
    assert (got.double() - oracle.gelu_tanh(gate.double()) * table[ids.long(), 8:12].double()).abs().max().item() < 1e-6


def test_layer_runs_caches_and_state(tmp_path_factory):
    """Every pass of a looped layer owns its cache rows and its state tensors; the weights (sinks among them) exist
    once; the recurrent state is fp32, the convolution tails are in the model dtype."""
    import types
    from vllm_distributed_amd.entrypoints import trace_replay
    from vllm_distributed_amd.models.gosizen import layer_runs
    assert [tuple(r) for r in layer_runs(4, {"start": 1, "stop": 3, "times": 2})] == \
        [(0, 0, -1), (1, 0, 0), (2, 0, -1), (1, 1, 1), (2, 1, -1), (3, 0, -1)]
    assert [tuple(r) for r in layer_runs(2, None)] == [(0, 0, -1), (1, 0, -1)]
    with pytest.raises(ValueError):
        layer_runs(3, {"start": 2, "stop": 4, "times": 2})
    path, cfg, w = model_dir("varied", tmp_path_factory)
    args = types.SimpleNamespace(model=path, dtype="bfloat16", out="", max_tokens=64, max_seqs=3, device="cpu",
                                 block_size=16, enforce_eager=True)
    core = trace_replay.make_core(args)
    try:
        mr = core.executor.driver.worker.model_runner
        model = mr.model
        owners = model.attention_layers()
        assert len(owners) == 1 + 2 * 3 + 1 and len({id(a) for a in owners}) == len(owners)
        assert owners[1].sink is owners[3].sink and owners[1].k_cache is not owners[3].k_cache
        assert len({a.k_cache.data_ptr() for a in owners}) == len(owners)
        names = [n for n, _ in model.named_parameters()]
        assert len(names) == len(set(names)) and sum(n.endswith("sink") for n in names) == 4
        states = model.state_layers()
        assert len(states) == 3 * (1 + 3) and len({id(s) for s in states}) == len(states)
        assert [tuple(s.shape) for s in mr.state_tensors[:3]] == [(4, 2, 4 * 16 + 2 * 16 + 2 * 8), (4, 3, 2 * 2 * 8 + 4 * 12),
                                                                  (4, 4, 8, 12)]
        assert [s.dtype for s in mr.state_tensors[:3]] == [torch.bfloat16, torch.bfloat16, torch.float32]
        assert owners[0].chunk == 7 and owners[0].window == 7 and owners[1].window == 9 and owners[1].interleaved
        spec = mr.get_kv_cache_spec()
        assert spec.sliding_window == 9            # the widest mask: pages further back than that are given back
        assert spec.bytes_per_token == 2 * ((2 * 16 + 2 * 8) + 3 * ((24 + 8) + (3 * 8 + 3 * 16)) + (12 + 4))
    finally:
        core.shutdown()


def test_config_errors():
    from vllm_distributed_amd.models.gosizen import GosizenLayer
    f32 = torch.float32
    ok = parallel(left(2, 1, 16, 8, 3, 11, 16), right(2, 1, 8, 8, 4), 0.5, 0.5, dense(48))
    ranks = {"l0.mix.right.a1": (4, 32), "l0.mix.right.g1": (4, 32)}
    GosizenLayer(32, ok, 1e-5, 0, f32, 1, 4, ranks)
    with pytest.raises(ValueError):                                               # no tensor states the ranks
        GosizenLayer(32, ok, 1e-5, 0, f32, 1, 4, {})
    for change in (lambda c: c.__setitem__("type", "other"),
                   lambda c: c["mixer"]["left"].__setitem__("kv_heads", 3),
                   lambda c: c["mixer"]["left"]["rot"].__setitem__("dims", 18),
                   lambda c: c["mixer"]["right"].__setitem__("kv_heads", 4),
                   lambda c: c["mlp"].__setitem__("kind", "other")):
        bad = json.loads(json.dumps(ok))
        change(bad)
        with pytest.raises(ValueError):
            GosizenLayer(32, bad, 1e-5, 0, f32, 1, 4, ranks)
    with pytest.raises(ValueError):                                               # an odd number of rotated values
        GosizenLayer(32, latent(2, 8, 8, 8, 16, 16, 6, None) | {"mixer": dict(latent(2, 8, 8, 8, 16, 16, 6)["mixer"], rot={"base": 10.0, "dims": 5})},
                     1e-5, 0, f32, 1, 0, {})


def test_dummy_weights_and_config_keys():
    """Random-weight loading (the benchmark's path): every parameter is filled, the derived keys are there."""
    from vllm_distributed_amd.config import normalize_hf_config
    from vllm_distributed_amd.models.gosizen import weight_shapes
    cfg = json.loads(json.dumps(CONFIGS["paged"]))
    for spec in cfg["layers"]:
        if spec["type"] == "parallel":
            spec["mixer"]["right"].update(decay_rank=5, gate_rank=7)
    shapes = weight_shapes(cfg)
    assert shapes["l1.mix.right.a2"] == (4 * 16, 5) and shapes["l1.mix.right.g1"] == (7, 64)
    assert shapes["loop.in"] == (64, 128) and shapes["side.embed"] == (97, 12) and shapes["l2.mlp.e3.down"] == (64, 32)
    n = dict(cfg)
    normalize_hf_config(n)
    assert n["hidden_size"] == 64 and n["vocab_size"] == 97 and n["num_hidden_layers"] == 3
    assert n["architectures"] == ["GosizenForCausalLM"]


def test_the_trace_runner_as_a_program(tmp_path_factory, tmp_path):
    import subprocess
    import sys
    path, cfg, w = model_dir("plain", tmp_path_factory)
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
    want = oracle_logits("plain", cfg, w, a)
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
