"""Nalasun in float64, written from the equations: one function per mechanism, loops over time wherever the design
has a recurrence or a convolution, whole score matrices for attention.  No code is shared with the package.
``w``: checkpoint tensor name -> tensor (any float type; read as float64)."""
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(h, taps_w, bias=None):
    """``h[T, C]``, ``taps_w[C, taps]`` (newest tap last); taps that reach in front of the first token add nothing."""
    t, taps = h.shape[0], taps_w.shape[1]
    y = torch.zeros_like(h)
    for i in range(t):
        for j in range(taps):
            src = i - (taps - 1) + j
            if src >= 0:
                y[i] += taps_w[:, j] * h[src]
    return y if bias is None else y + bias


def q_temperature(positions, coef, every):
    return 1.0 + coef * torch.log(torch.floor((positions.to(F64) + 1.0) / every) + 1.0)


def softmax_weights(q, k, scale, r1, r2):
    """``q[T, H, D]``, ``k[T, G, D]`` -> causal softmax weights ``[H, T, T]`` with the distance bias taken off."""
    t, heads, groups = q.shape[0], q.shape[1], k.shape[1]
    i = torch.arange(t).view(-1, 1)
    j = torch.arange(t).view(1, -1)
    dist = (i - j).clamp(min=0).to(F64)
    out = torch.zeros(heads, t, t, dtype=F64)
    for h in range(heads):
        s = (q[:, h] @ k[:, h // (heads // groups)].T) * scale - r1[h] * torch.log(1.0 + r2[h] * dist)
        out[h] = torch.softmax(s.masked_fill(j > i, float("-inf")), dim=-1)
    return out


def attention_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, groups, dim = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"])
    q = h @ f64(w[p + "q"]).T + f64(w[p + "q.b"])
    k = h @ f64(w[p + "k"]).T + f64(w[p + "k.b"])
    values = k.view(t, groups, dim)                                        # the un-normed key projection
    q = unit_rms(q, eps) * f64(w[p + "q.norm"])                            # jointly over all heads
    k = unit_rms(k, eps) * f64(w[p + "k.norm"])
    if m.get("q_temp"):
        q = q * q_temperature(torch.arange(t), float(m["q_temp"]["coef"]), int(m["q_temp"]["every"])).view(-1, 1)
    weights = softmax_weights(q.view(t, heads, dim), k.view(t, groups, dim), float(m["scale"]), f64(w[p + "r1"]),
                              f64(w[p + "r2"]))
    mixed = torch.einsum("hg,gij->hij", f64(w[p + "talk"]), weights)
    o = torch.stack([mixed[hh] @ values[:, hh // (heads // groups)] for hh in range(heads)], dim=1)
    return o.reshape(t, heads * dim) @ f64(w[p + "o"]).T


def delta_heads(q, k, v, beta, decay, state=None):
    """``q, k[T, H, D]`` (unit vectors, q scaled), ``v[T, H, V]``, ``beta[T, H]``, ``decay[T, H, D]`` -> outputs
    ``[T, H, V]`` and the final state ``[H, D, V]``."""
    t, heads, dim = q.shape
    vdim = v.shape[2]
    s = torch.zeros(heads, dim, vdim, dtype=F64) if state is None else state.clone()
    out = torch.zeros(t, heads, vdim, dtype=F64)
    for i in range(t):
        for h in range(heads):
            s[h] = decay[i, h].view(-1, 1) * s[h]
            u = beta[i, h] * (v[i, h] - s[h].T @ k[i, h])
            s[h] = s[h] + torch.outer(k[i, h], u)
            out[i, h] = s[h].T @ q[i, h]
    return out, s


def channel_delta_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, groups = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
    dim, vdim = int(m["dim"]), int(m.get("vdim") or m["dim"])
    q = silu(causal_conv(h @ f64(w[p + "q"]).T, f64(w[p + "q.conv"]))).view(t, groups, dim)
    k = silu(causal_conv(h @ f64(w[p + "k"]).T, f64(w[p + "k.conv"]))).view(t, groups, dim)
    v = silu(causal_conv(h @ f64(w[p + "v"]).T, f64(w[p + "v.conv"]))).view(t, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = heads // groups
    beta = sigmoid(h @ f64(w[p + "b"]).T)
    dt = (h @ f64(w[p + "a1"]).T) @ f64(w[p + "a2"]).T + f64(w[p + "dt_bias"])
    decay = torch.exp(-torch.exp(f64(w[p + "A_log"])).view(1, heads, 1) * softplus(dt).view(t, heads, dim))
    o, _ = delta_heads(q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1), v, beta, decay)
    gate = sigmoid((h @ f64(w[p + "g1"]).T) @ f64(w[p + "g2"]).T).view(t, heads, vdim)
    o = unit_rms(o, eps) * f64(w[p + "norm"]) * gate
    return o.reshape(t, heads * vdim) @ f64(w[p + "o"]).T


def ssm_heads(x, b, c, step, rate, skip, state=None):
    """``x[T, H, V]``, ``b, c[T, H, N]``, ``step[T, H]`` (after softplus), ``rate[H]`` = exp(A_log), ``skip[H]`` ->
    outputs ``[T, H, V]`` and the final state ``[H, N, V]``."""
    t, heads, vdim = x.shape
    n = b.shape[2]
    s = torch.zeros(heads, n, vdim, dtype=F64) if state is None else state.clone()
    y = torch.zeros(t, heads, vdim, dtype=F64)
    for i in range(t):
        for h in range(heads):
            s[h] = torch.exp(-rate[h] * step[i, h]) * s[h] + step[i, h] * torch.outer(b[i, h], x[i, h])
            y[i, h] = s[h].T @ c[i, h] + skip[h] * x[i, h]
    return y, s


def mamba2_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, vdim, n, groups = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups") or 1)
    inner, parts = heads * vdim, int(m.get("norm_groups") or 1)
    u = h @ f64(w[p + "in"]).T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * groups * n], u[:, 2 * inner + 2 * groups * n:]
    xbc = silu(causal_conv(xbc, f64(w[p + "conv"]), f64(w[p + "conv.b"])))
    rep = heads // groups
    x = xbc[:, :inner].view(t, heads, vdim)
    b = xbc[:, inner:inner + groups * n].view(t, groups, n).repeat_interleave(rep, 1)
    c = xbc[:, inner + groups * n:].view(t, groups, n).repeat_interleave(rep, 1)
    y, _ = ssm_heads(x, b, c, softplus(dt + f64(w[p + "dt_bias"])), torch.exp(f64(w[p + "A_log"])), f64(w[p + "D"]))
    y = y.reshape(t, inner) * silu(z)                                     # gated first, normed second
    y = unit_rms(y.view(t, parts, inner // parts), eps).reshape(t, inner) * f64(w[p + "norm"])
    return y @ f64(w[p + "o"]).T


def expert(h, w, p):
    return (silu(h @ f64(w[p + "gate"]).T) * (h @ f64(w[p + "up"]).T)) @ f64(w[p + "down"]).T


def route(h, w, p, top, scale):
    """Chosen experts ``[T, top]`` and their weights: the sigmoid scores themselves, times ``scale``."""
    s = sigmoid(h @ f64(w[p + "router"]).T)
    idx = torch.topk(s, top, dim=-1).indices
    return idx, s.gather(1, idx) * scale


def moe_ff(h, w, p, mlp):
    r = mlp["router"]
    idx, wts = route(h, w, p, int(r["top"]), float(r.get("scale", 1.0)))
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for j, e in enumerate(idx[i].tolist()):
            out[i] += wts[i, j] * expert(h[i:i + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + expert(h, w, p + "shared.")
    return out


MIXERS = {"attention": attention_mixer, "channel_delta": channel_delta_mixer, "mamba2": mamba2_mixer}


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None):
    """Logits ``[T, vocab]`` of a whole sequence; ``residuals`` collects the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    t = len(tokens)
    x = f64(w["embed"])[tokens] + f64(w["pos"])[:t]
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = unit_rms(x, eps) * f64(w[p + "norm1"])
        if (cfg.get("canon") or {}).get("taps"):
            h = h + causal_conv(h, f64(w[p + "canon1"]))
        x = x + MIXERS[spec["type"]](h, w, p + "mix.", spec["mixer"], eps)
        if spec.get("mlp"):
            x = x + moe_ff(unit_rms(x, eps) * f64(w[p + "norm2"]), w, p + "mlp.", spec["mlp"])
        if residuals is not None:
            residuals.append(x.clone())
    return (unit_rms(x, eps) * f64(w["final.norm"])) @ f64(w["embed"]).T
