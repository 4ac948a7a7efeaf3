"""A plain, slow implementation of the Talolorn decoder: whole sequences, no cache, one
function per mechanism, written from the design's equations and sharing no code with the
package (it reads a model folder through the ``safetensors`` package).

Notation: x is the residual stream [T, width]; a layer computes h = rmsnorm(x) * g and
x <- x + m * (mixer(h) + ff(h)).  Linear weights are stored [out, in] and applied as W h.
`cast` rounds a tensor the way a bfloat16 run rounds what it stores between two products
(identity for a float32 or float64 run); accumulation is in the working precision.
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


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def rotate_interleaved(x, positions, base, dims):
    """x [..., T, n]: the first `dims` dims turn, pair i = dims (2i, 2i+1) by the angle
    p * base^(-2i/dims); the rest passes unchanged.  positions [T]."""
    out = x.clone()
    if dims == 0:
        return out
    i = torch.arange(dims // 2, dtype=torch.float32)
    freq = base ** (-2.0 * i / dims)
    angle = positions.to(torch.float32)[:, None] * freq[None, :]
    cos, sin = angle.cos().to(x.dtype), angle.sin().to(x.dtype)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def gate_activation(g, u, limit):
    """g' * sigmoid(1.702 g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit)."""
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def dense_ff(h, w, prefix, ff, cast=identity):
    act = cast(gate_activation(cast(h @ w[prefix + "gate"].T), cast(h @ w[prefix + "up"].T), ff["limit"]))
    return act @ w[prefix + "down"].T


def route(h, router_weight, experts, top, scale):
    """Scores softmax(W h) over all experts; the `top` largest (ties: lower index) with their
    scores times `scale`, not renormalised.  Returns (indices [T, top], weights [T, top])."""
    scores = torch.softmax((h.float() @ router_weight.float().T), dim=-1)
    chosen = torch.zeros(h.shape[0], top, dtype=torch.long)
    weights = torch.zeros(h.shape[0], top)
    for t in range(h.shape[0]):
        left = scores[t].clone()
        for j in range(top):
            e = int(torch.argmax(left))        # the first of equals
            chosen[t, j], weights[t, j] = e, scores[t, e] * scale
            left[e] = -1.0
    return chosen, weights


def routing_gap(h, router_weight, top):
    """Per token: how far the last chosen score stands above the first one not chosen, as a
    fraction of it (inf when every expert is chosen).  A small gap is a close call that
    rounding may decide the other way."""
    scores = torch.softmax((h.float() @ router_weight.float().T), dim=-1)
    ordered = torch.sort(scores, dim=-1, descending=True).values
    if top >= ordered.shape[-1]:
        return torch.full((h.shape[0],), math.inf)
    return (ordered[:, top - 1] - ordered[:, top]) / ordered[:, top - 1]


def routed_ff(h, w, prefix, ff, cast=identity, gaps=None):
    r = ff["router"]
    chosen, weights = route(h, w[prefix + "router"], r["experts"], r["top"], r["scale"])
    if gaps is not None:
        gaps.append(routing_gap(h, w[prefix + "router"], r["top"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(r["top"]):
            e = int(chosen[t, j])
            out[t] += weights[t, j].to(h.dtype) * dense_ff(h[t:t + 1], w, f"{prefix}e{e}.", ff["expert"], cast)[0]
    return out


def latent_attention(h, w, prefix, m, eps, cast=identity, positions=None):
    """The mixer over a whole sequence (position i sees every j <= i), keys and values of
    every head written out from the latent."""
    T = h.shape[0]
    H, d, r, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = torch.arange(T) if positions is None else positions
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    c_q = cast(rms_norm(h @ w[prefix + "dq"].T, w[prefix + "dq.norm"], eps))
    q = cast(c_q @ w[prefix + "uq"].T).view(T, H, d + r)
    down = h @ w[prefix + "dkv"].T
    c = cast(rms_norm(down[:, :rank], w[prefix + "dkv.norm"], eps))
    shared = cast(rotate_interleaved(down[:, rank:], positions, base, dims))      # [T, r]
    k_plain = cast(c @ w[prefix + "uk"].T).view(T, H, d)
    v = cast(c @ w[prefix + "uv"].T).view(T, H, vd)
    q_plain = q[..., :d]
    q_rot = cast(rotate_interleaved(q[..., d:].transpose(0, 1), positions, base, dims))  # [H, T, r]
    out = torch.zeros(T, H, vd, dtype=h.dtype)
    for head in range(H):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_rot[head] @ shared.T) * m["scale"]
        score = score.float()
        score = score.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
        p = torch.softmax(score, dim=-1).to(h.dtype)
        out[:, head] = p @ v[:, head]
    return cast(out.reshape(T, H * vd)) @ w[prefix + "o"].T


def feed_forward(h, w, prefix, ff, cast=identity, gaps=None):
    if ff is None:
        return torch.zeros_like(h)
    if ff["kind"] == "dense":
        return dense_ff(h, w, prefix, ff, cast)
    return routed_ff(h, w, prefix, ff, cast, gaps)


def layer(x, w, cfg, index, cast=identity, gaps=None):
    entry = cfg["layers"][index]
    owner = entry.get("weights_of", index)
    eps = cfg["norm"]["eps"]
    h = cast(rms_norm(x, w[f"l{owner}.norm1"], eps))
    mixed = latent_attention(h, w, f"l{owner}.mix.", entry["mixer"], eps, cast)
    return x + cfg["residual_mult"] * (mixed + feed_forward(h, w, f"l{owner}.mlp.", entry["mlp"], cast, gaps))


def forward_logits(w, cfg, tokens, cast=identity, streams=None, gaps=None):
    """Logits [T, vocab] of a whole sequence; `streams`, a list, receives the residual stream
    after every layer, `gaps`, a list, every routed layer's routing gaps [T]."""
    x = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for index in range(len(cfg["layers"])):
        x = layer(x, w, cfg, index, cast, gaps)
        if streams is not None:
            streams.append(x.clone())
    return cast(rms_norm(x, w["final.norm"], cfg["norm"]["eps"])) @ w["head"].T


def greedy_generate(w, cfg, prompt, count):
    tokens, out = list(prompt), []
    for _ in range(count):
        out.append(int(torch.argmax(forward_logits(w, cfg, tokens)[-1])))
        tokens.append(out[-1])
    return out
