"""A plain, slow implementation of the Larozen decoder: whole sequences, no cache, one
function per mechanism, written from the design's equations and sharing no code with the
package (it reads a model folder through the ``safetensors`` package).

Notation: s is the residual stream [T, width], e the embedding output.  A layer computes
s <- s + mixer(n1(s)), s <- s + ff(n2(s)) with n(s) = s / rms(s) * (1 + g).  Linear weights
are stored [out, in] and applied as W h.  `cast` rounds a tensor the way a bfloat16 run rounds
what it hands from one product to the next (identity for a float32 or float64 run).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def read_weights(folder, dtype=torch.float32) -> dict:
    from safetensors.torch import load_file

    return {k: v.to(dtype) for k, v in load_file(str(Path(folder) / "model.safetensors")).items()}


def identity(t):
    return t


def to_bf16(t):
    return t.to(torch.bfloat16).to(t.dtype)


# ---------------------------------------------------------------------------- mechanisms


def rms(x, eps):
    """Root mean square over the last axis, eps inside the root."""
    return torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, g, eps):
    """The layer norms and the final norm: the stored weight lies around zero."""
    return x / rms(x, eps) * (1.0 + g)


def norm_plain(x, g, eps):
    return x / rms(x, eps) * g


def turn_pairs(x, positions, base, dims):
    """x [T, heads, n]: of every head the first `dims` entries turn, entries 2i and 2i+1
    together by the angle p * base^(-2i/dims); the others stay."""
    out = x.clone()
    if not dims:
        return out
    i = torch.arange(dims // 2, dtype=torch.float64)
    angle = positions.to(torch.float64)[:, None] * (float(base) ** (-2.0 * i / dims))[None, :]
    cos, sin = angle.cos().to(x.dtype)[:, None, :], angle.sin().to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def query_temperature(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1) per position."""
    steps = torch.div(positions.to(torch.int64) + 1, int(every), rounding_mode="floor")
    return 1.0 + coef * torch.log(steps.to(torch.float64) + 1.0)


def causal_weights(q, k, scale, softcap=None, sink=None):
    """q [T, H, d], k [T, G, d] -> attention weights [H, T, T] over j <= i.  `softcap` c
    bounds the scaled score to c tanh(score / c).  `sink` [H]: exp(sink_h) stands in the
    denominator once, unscaled, with no key or value behind it."""
    T, H, _ = q.shape
    G = k.shape[1]
    k = k.repeat_interleave(H // G, dim=1)
    score = torch.einsum("ihd,jhd->hij", q, k) * scale
    if softcap:
        score = softcap * torch.tanh(score / softcap)
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    score = score.masked_fill(~mask, float("-inf"))
    if sink is None:
        return torch.softmax(score, dim=-1)
    top = torch.maximum(score.max(-1, keepdim=True).values, sink.to(score.dtype)[:, None, None])
    e = torch.exp(score - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink.to(score.dtype)[:, None, None] - top))


def weighted_values(p, v):
    """p [H, T, T], v [T, G, dv] -> [T, H * dv]."""
    H, G = p.shape[0], v.shape[1]
    v = v.repeat_interleave(H // G, dim=1)
    return torch.einsum("hij,jhd->ihd", p, v).reshape(p.shape[1], -1)


def attention_mixer(h, w, prefix, m, positions, cast=identity):
    """Rotated queries and keys with a capped score; the values are the keys as projected."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[prefix + "q"].T + w[prefix + "q.b"]).view(T, H, d)
    k = (h @ w[prefix + "k"].T + w[prefix + "k.b"]).view(T, G, d)
    v = cast(k)
    rot = m.get("rot") or {}
    q = cast(turn_pairs(q, positions, rot.get("base", 1.0), rot.get("dims", 0)))
    kr = cast(turn_pairs(k, positions, rot.get("base", 1.0), rot.get("dims", 0)))
    p = causal_weights(q, kr, m["scale"], softcap=m.get("softcap"))
    return cast(weighted_values(p, v)) @ w[prefix + "o"].T


def sink_attention(h, w, prefix, m, positions, eps, cast=identity):
    """The left half of a parallel mixer: q and k normed over the whole projection, queries
    scaled with the position, a sink in the softmax, biases everywhere, no rotation."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[prefix + "q"].T + w[prefix + "q.b"]
    k = h @ w[prefix + "k"].T + w[prefix + "k.b"]
    v = cast(h @ w[prefix + "v"].T + w[prefix + "v.b"]).view(T, G, dv)
    q = norm_plain(q, w[prefix + "q.norm"], eps)
    k = norm_plain(k, w[prefix + "k.norm"], eps)
    temp = m.get("q_temp")
    if temp:
        q = q * query_temperature(positions, temp["coef"], temp["every"]).to(q.dtype)[:, None]
    q, k = cast(q).view(T, H, d), cast(k).view(T, G, d)
    p = causal_weights(q, k, m["scale"], sink=w[prefix + "sink"])
    return cast(weighted_values(p, v)) @ w[prefix + "o"].T + w[prefix + "o.b"]


def causal_conv(u, weight, bias):
    """u [T, C], weight [C, taps] whose last column meets the current token; zeros before the
    sequence."""
    T, C = u.shape
    taps = weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], dim=0)
    out = bias.to(u.dtype).expand(T, C).clone()
    for j in range(taps):
        out = out + padded[j:j + T] * weight[:, j]
    return out


def silu(x):
    return x * torch.sigmoid(x)


def state_space(x, B, C, dt, A_log, D, heads, groups):
    """x [T, heads, P], B and C [T, groups, N], dt [T, heads] (after its softplus).  Per head
    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t; S starts
    at zero."""
    T, _, P = x.shape
    N = B.shape[-1]
    per = heads // groups
    S = torch.zeros(heads, N, P, dtype=x.dtype)
    rate = torch.exp(A_log.to(x.dtype))
    y = torch.zeros_like(x)
    for t in range(T):
        Bt = B[t].repeat_interleave(per, dim=0)
        Ct = C[t].repeat_interleave(per, dim=0)
        decay = torch.exp(-rate * dt[t])
        S = decay[:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, Ct) + D.to(x.dtype)[:, None] * x[t]
    return y


def state_space_mixer(h, w, prefix, m, eps, cast=identity):
    """The right half of a parallel mixer."""
    T = h.shape[0]
    heads, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * P
    proj = h @ w[prefix + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[prefix + "conv"], w[prefix + "conv.b"]))
    x = xbc[:, :inner].view(T, heads, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[prefix + "dt_bias"], threshold=1e9)
    y = state_space(x, B, C, dt, w[prefix + "A_log"], w[prefix + "D"], heads, G).reshape(T, inner)
    y = y * silu(z)
    parts = m["norm_groups"]
    y = y.view(T, parts, inner // parts)
    y = (y / rms(y, eps)).reshape(T, inner) * w[prefix + "norm"]
    return cast(y) @ w[prefix + "o"].T


def parallel_mixer(h, w, prefix, m, positions, eps, cast=identity):
    left = sink_attention(h, w, prefix + "left.", m["left"], positions, eps, cast)
    right = state_space_mixer(h, w, prefix + "right.", m["right"], eps, cast)
    return 0.5 * (norm_plain(left, w[prefix + "left.out"], eps)
                  + norm_plain(right, w[prefix + "right.out"], eps))


def squared_relu_ff(h, w, prefix, cast=identity):
    up = torch.relu(h @ w[prefix + "up"].T)
    return cast(up * up) @ w[prefix + "down"].T


# --------------------------------------------------------------------------------- model


def layer_order(cfg):
    """The layers in the order they run: (layer index, first of a pass?)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg, w, tokens, cast=identity, keep_layers=False):
    """Logits [T, vocab] of one sequence; with keep_layers also the stream after every layer
    run.  `w` in the working precision (float32 or float64)."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    s = w["embed"][tokens]
    e = s
    kept = []
    for i, first in layer_order(cfg):
        entry = cfg["layers"][i]
        p = f"l{i}."
        if first:
            s = cast(torch.cat([s, e], dim=-1)) @ w["loop.in"].T
        h = cast(norm_one_plus(s, w[p + "norm1"], eps))
        if entry["type"] == "attention":
            s = s + attention_mixer(h, w, p + "mix.", entry["mixer"], positions, cast)
        elif entry["type"] == "parallel":
            s = s + parallel_mixer(h, w, p + "mix.", entry["mixer"], positions, eps, cast)
        else:
            raise ValueError(entry["type"])
        if entry.get("mlp"):
            h = cast(norm_one_plus(s, w[p + "norm2"], eps))
            s = s + squared_relu_ff(h, w, p + "mlp.", cast)
        if keep_layers:
            kept.append(s.clone())
    logits = cast(norm_one_plus(s, w["final.norm"], eps)) @ w["embed"].T
    return (logits, torch.stack(kept)) if keep_layers else logits
