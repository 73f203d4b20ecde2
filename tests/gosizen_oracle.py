"""Gosizen in float64, written from the equations: one function per mechanism, loops over positions where the model
is a recurrence, whole ``[T, T]`` score matrices where it is attention.  Shares no code with the package; the tests
compare the framework against it.

Weights: a dict of tensors under the checkpoint's names (any float type; used as float64).
"""
import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the gain minus one."""
    return unit_rms(x, eps) * (1 + f64(w))


def sigmoid(x):
    return 1 / (1 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2)))


# ------------------------------------------------------------------------------------------------ rotations
def frequencies(rot):
    """``f_i = base^(-2i / dims)``; with ``scaling`` the long wavelengths are slowed down by ``factor``, the short
    ones kept, and those between blended linearly in ``original / wavelength``."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        out = []
        for x in f:
            wavelength = 2 * math.pi / x
            if wavelength < sc["original"] / sc["high"]:
                out.append(x)
            elif wavelength > sc["original"] / sc["low"]:
                out.append(x / sc["factor"])
            else:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1 - s) * x / sc["factor"] + s * x)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate(x, positions, rot, interleaved):
    """``x[T, ..., n]``: the first ``rot.dims`` values of the last axis turn by ``position * f_i``; pair ``i`` is
    values ``(2i, 2i + 1)`` when ``interleaved``, else ``(i, i + dims / 2)``."""
    dims = rot["dims"]
    half = dims // 2
    f = frequencies(rot)
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(half):
            a = float(positions[t]) * float(f[i])
            c, s = math.cos(a), math.sin(a)
            iu, iv = (2 * i, 2 * i + 1) if interleaved else (i, i + half)
            u, v = x[t, ..., iu], x[t, ..., iv]
            out[t, ..., iu] = u * c - v * s
            out[t, ..., iv] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ attention
def window_mask(positions, size):
    """[T, T] true where query i sees key j: itself and the ``size - 1`` tokens before it."""
    i, j = positions.view(-1, 1), positions.view(1, -1)
    return (j <= i) & (i - j < size)


def chunk_mask(positions, size):
    """[T, T] true where query i sees key j: j <= i in the same block of ``size`` positions counted from 0."""
    i, j = positions.view(-1, 1), positions.view(1, -1)
    return (j <= i) & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))


def sink_softmax(scores, seen, sink):
    """Softmax over the seen keys of ``scores[T, T]`` with ``exp(sink)`` added to the denominator."""
    t = scores.shape[0]
    p = torch.zeros_like(scores)
    for i in range(t):
        idx = torch.nonzero(seen[i]).flatten()
        s = scores[i, idx]
        m = max(float(s.max()), float(sink))
        e = torch.exp(s - m)
        p[i, idx] = e / (e.sum() + math.exp(float(sink) - m))
    return p


def latent_attention(h, w, p, m, eps, positions):
    t = h.shape[0]
    heads, dim, rd, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = unit_rms(h @ f64(w[p + "dq"]).T, eps) * f64(w[p + "dq.norm"])
    q = (cq @ f64(w[p + "uq"]).T).view(t, heads, dim + rd)
    down = h @ f64(w[p + "dkv"]).T
    c = unit_rms(down[:, :rank], eps) * f64(w[p + "dkv.norm"])
    k_rot = rotate(down[:, rank:], positions, m["rot"], True)
    q_rot = rotate(q[..., dim:], positions, m["rot"], True)
    k_un = (c @ f64(w[p + "uk"]).T).view(t, heads, dim)
    v = (c @ f64(w[p + "uv"]).T).view(t, heads, vd)
    seen = window_mask(positions, m["mask"]["size"])
    gate = sigmoid(h @ f64(w[p + "g"]).T)
    out = torch.zeros(t, heads, vd, dtype=F64)
    for hh in range(heads):
        s = (q[:, hh, :dim] @ k_un[:, hh].T + q_rot[:, hh] @ k_rot.T) * m["scale"]
        out[:, hh] = sink_softmax(s, seen, f64(w[p + "sink"])[hh]) @ v[:, hh] * gate[:, hh:hh + 1]
    return out.reshape(t, heads * vd) @ f64(w[p + "o"]).T


def causal_conv(u, w):
    """``u[T, C]``, ``w[C, taps]`` (last column: the current token's), zeros before the start."""
    t, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for i in range(t):
        for j in range(taps):
            src = i - taps + 1 + j
            if src >= 0:
                y[i] += f64(w)[:, j] * u[src]
    return y


def chunked_attention(h, w, p, m, positions):
    t = h.shape[0]
    heads, kvh, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv(h @ f64(w[p + "q"]).T + f64(w[p + "q.b"]), w[p + "q.conv"]).view(t, heads, dim)
    k = causal_conv(h @ f64(w[p + "k"]).T + f64(w[p + "k.b"]), w[p + "k.conv"]).view(t, kvh, dim)
    v = causal_conv(h @ f64(w[p + "v"]).T + f64(w[p + "v.b"]), w[p + "v.conv"]).view(t, kvh, vd)
    q, k = rotate(q, positions, m["rot"], False), rotate(k, positions, m["rot"], False)
    seen = chunk_mask(positions, m["mask"]["size"])
    out = torch.zeros(t, heads, vd, dtype=F64)
    for hh in range(heads):
        g = hh // (heads // kvh)
        s = q[:, hh] @ k[:, g].T * m["scale"]
        out[:, hh] = sink_softmax(s, seen, f64(w[p + "sink"])[hh]) @ v[:, g]
    out = out.reshape(t, heads * vd) * sigmoid(h @ f64(w[p + "g"]).T)
    return out @ f64(w[p + "o"]).T


# ------------------------------------------------------------------------------------------------ gated delta rule
def delta_heads(q, k, v, beta, decay, state=None):
    """``q, k [T, H, dk]`` (unit vectors, q scaled), ``v [T, H, dv]``, ``beta [T, H]``, ``decay [T, H, dk]``: per head
    ``S <- decay * S`` by rows, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``.  Returns (o, final S)."""
    t, h, dk = q.shape
    dv = v.shape[2]
    s = torch.zeros(h, dk, dv, dtype=F64) if state is None else state.clone()
    o = torch.zeros(t, h, dv, dtype=F64)
    for i in range(t):
        for hh in range(h):
            s[hh] = decay[i, hh].view(dk, 1) * s[hh]
            u = beta[i, hh] * (v[i, hh] - s[hh].T @ k[i, hh])
            s[hh] = s[hh] + torch.outer(k[i, hh], u)
            o[i, hh] = s[hh].T @ q[i, hh]
    return o, s


def delta_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, kvh, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ f64(w[p + "q"]).T, w[p + "q.conv"])).view(t, kvh, dim)
    k = silu(causal_conv(h @ f64(w[p + "k"]).T, w[p + "k.conv"])).view(t, kvh, dim)
    v = silu(causal_conv(h @ f64(w[p + "v"]).T, w[p + "v.conv"])).view(t, heads, vd)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = heads // kvh
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)
    beta = sigmoid(h @ f64(w[p + "b"]).T)
    dt = softplus((h @ f64(w[p + "a1"]).T) @ f64(w[p + "a2"]).T + f64(w[p + "dt_bias"])).view(t, heads, dim)
    decay = torch.exp(-torch.exp(f64(w[p + "A_log"])).view(1, heads, 1) * dt)
    o, _ = delta_heads(q, k, v, beta, decay)
    o = unit_rms(o, eps) * f64(w[p + "norm"])
    o = o.reshape(t, heads * vd) * sigmoid((h @ f64(w[p + "g1"]).T) @ f64(w[p + "g2"]).T)
    return o @ f64(w[p + "o"]).T


def parallel_mixer(h, w, p, m, eps, positions):
    return (m["left_scale"] * chunked_attention(h, w, p + "left.", m["left"], positions)
            + m["right_scale"] * delta_mixer(h, w, p + "right.", m["right"], eps))


# ------------------------------------------------------------------------------------------------ feed-forwards
def dense_ff(h, w, p):
    return gelu_tanh(h @ f64(w[p + "up"]).T) @ f64(w[p + "down"]).T


def route(h, w, p, top):
    """Per token the ``top`` largest router logits and the softmax over just those."""
    z = h @ f64(w[p + "router"]).T + f64(w[p + "router.b"])
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, -1)


def moe_ff(h, w, p, mlp):
    idx, wt = route(h, w, p, mlp["router"]["top"])
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = f"{p}e{int(idx[t, j])}."
            out[t] += wt[t, j] * (gelu_erf(h[t] @ f64(w[e + "up"]).T) @ f64(w[e + "down"]).T)
    return out


def token_side(x, tokens, w, p, layer, dim, eps):
    e = f64(w["side.embed"])[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ f64(w[p + "side.gate"]).T) * e) @ f64(w[p + "side.proj"]).T
    return unit_rms(y, eps) * f64(w[p + "side.norm"])


# ------------------------------------------------------------------------------------------------ the model
def layer_runs(cfg):
    """The layers in the order they run, as (layer index, pass number or None, first of its pass)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None, False) for i in range(loop["stop"], n)]


def forward(cfg, w, tokens, trace=None):
    """Logits ``[T, vocab]`` of one sequence from position 0; ``trace`` (a list) receives the residual stream after
    every layer run."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    eps = cfg["norm"]["eps"]
    x = f64(w["embed"])[tokens]
    x0 = x.clone()
    side = (cfg.get("token_side") or {}).get("dim")
    for i, t, first in layer_runs(cfg):
        spec, p = cfg["layers"][i], f"l{i}."
        if first:
            x = torch.cat([x, x0], -1) @ f64(w["loop.in"]).T + f64(w["loop.step"])[t]
        h = offset_norm(x, w[p + "norm1"], eps)
        if spec["type"] == "latent_attention":
            y = latent_attention(h, w, p + "mix.", spec["mixer"], eps, positions)
        elif spec["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", spec["mixer"], eps, positions)
        else:
            raise ValueError(spec["type"])
        mlp = spec.get("mlp")
        if mlp:
            y = y + (dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, w, p + "mlp.", mlp))
        x = x + y
        if side:
            x = x + token_side(x, tokens, w, p, i, side, eps)
        if trace is not None:
            trace.append(x.clone())
    y = offset_norm(x, w["final.norm"], eps) @ f64(w["head"]).T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(y / cap) if cap else y
