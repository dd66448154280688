"""The plain Nevodra model: one function per mechanism, written from the design's equations, whole sequences at once,
no cache, no batching, float64 by default. It shares no code with the engine; the tests hold the engine to it.

Notation: x [n, W] the residual stream of a sequence of n tokens at positions 0 .. n - 1; `w` maps checkpoint tensor
names to tensors; `p` is a tensor name prefix.

  rms(v)          v / sqrt(mean(v^2) + eps), over the last dimension
  layer           x <- x + mixer(F1(rms(x) g1)) + ffn(F2(rms(x) g2)),  F(a)_t = a_t + sum_j c[:, j] a_(t - taps + 1 + j)
  attention       q = rms_all(Wq a) gq, k = rms_all(Wk a) gk (one norm over the whole projection), v = Wv a;
                  s_ij = cap tanh(scale q_i . k_j / cap) - r1 ln(1 + r2 (i - j));  j visible if j <= i and
                  (i - j < size or j < keep_first); softmax; Wo on the heads side by side
  latent          q = Wq a, per head [dim plain, rot turned]; [c', kr] = Wdkv a, c = rms(c') gc; k_h = Wuk,h c,
                  v_h = Wuv,h c; s_ij = scale (q_plain . k_h + turn(q_rot, i) . turn(kr, j)); causal; softmax whose
                  denominator also holds exp(sink_h); Wo
  turn(u, p)      pairs (u_2i, u_2i+1), i < dims / 2, rotated by the angle p base^(-2i / dims)
  dense ffn       Wdown P(Wup a),  P(z) = a N(z) + b N(z^2) + c N(z^3) + e,  N(v) = v / sqrt(mean(v^2) + eps)
  experts         sum over chosen e of scale s_e Wdown,e (silu(Wgate,e a) * (Wup,e a)) + shared(a);  s = sigmoid(Wr a);
                  chosen: the `top` largest of s + correction among the experts of the `keep` groups (of `count`
                  groups of neighbours) whose two largest s + correction sum highest
  loop            layers start .. stop - 1 run `times` times; step[t] is added to x in front of pass t
"""
from __future__ import annotations

import math

import torch


def rms(v, eps):
    return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)


def causal_filter(a, taps_w):
    """a [n, W], taps_w [W, taps] -> a + conv(a), zeros before the sequence's start."""
    n, taps = a.shape[0], taps_w.shape[1]
    padded = torch.cat((a.new_zeros(taps - 1, a.shape[1]), a))
    out = a.clone()
    for j in range(taps):
        out = out + taps_w[:, j] * padded[j: j + n]
    return out


def visible(n, size, keep_first):
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    seen = j <= i
    if size:
        seen = seen & ((i - j < size) | (j < keep_first))
    return seen


def attention(w, p, m, a, eps):
    n = a.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    groups = m.get("kv_heads") or heads
    q = (rms(a @ w[p + "q"].T, eps) * w[p + "q.norm"]).view(n, heads, dim)
    k = (rms(a @ w[p + "k"].T, eps) * w[p + "k.norm"]).view(n, groups, dim)
    v = (a @ w[p + "v"].T).view(n, groups, vdim)
    mask = m.get("mask") or {}
    seen = visible(n, mask.get("size", 0), mask.get("keep_first", 0))
    out = a.new_zeros(n, heads, vdim)
    dist = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).clamp(min=0).to(a.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        s = (q[:, h] @ k[:, g].T) * m["scale"]
        if m.get("softcap"):
            s = m["softcap"] * torch.tanh(s / m["softcap"])
        s = s - w[p + "r1"][h] * torch.log1p(w[p + "r2"][h] * dist)
        s = s.masked_fill(~seen, -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out.reshape(n, heads * vdim) @ w[p + "o"].T


def turn(u, positions, base, dims):
    """u [n, ..., d]: the first `dims` dimensions in pairs (2i, 2i + 1) rotated by positions * base^(-2i / dims)."""
    if not dims:
        return u
    i = torch.arange(dims // 2, dtype=u.dtype)
    angle = positions.to(u.dtype)[:, None] * base ** (-2 * i / dims)
    shape = (u.shape[0],) + (1,) * (u.dim() - 2) + (dims // 2,)
    cos, sin = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
    even, odd = u[..., 0:dims:2], u[..., 1:dims:2]
    out = u.clone()
    out[..., 0:dims:2] = even * cos - odd * sin
    out[..., 1:dims:2] = odd * cos + even * sin
    return out


def latent_attention(w, p, m, a, eps):
    n = a.shape[0]
    heads, dim, vdim, rank, rot = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m.get("rot_dim", 0)
    q = (a @ w[p + "q"].T).view(n, heads, dim + rot)
    down = a @ w[p + "dkv"].T
    c = rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_plain = (c @ w[p + "uk"].T).view(n, heads, dim)
    v = (c @ w[p + "uv"].T).view(n, heads, vdim)
    positions = torch.arange(n)
    base, dims = (m["rot"]["base"], m["rot"]["dims"]) if rot else (1.0, 0)
    q_rot = turn(q[..., dim:], positions, base, dims)
    k_rot = turn(down[:, rank:], positions, base, dims)
    hidden = torch.arange(n)[None, :] > torch.arange(n)[:, None]
    out = a.new_zeros(n, heads, vdim)
    for h in range(heads):
        s = (q[:, h, :dim] @ k_plain[:, h].T + q_rot[:, h] @ k_rot.T) * m["scale"]
        s = s.masked_fill(hidden, -math.inf)
        top = torch.maximum(s.max(-1, keepdim=True).values, w[p + "sink"][h])
        e = torch.exp(s - top)
        out[:, h] = (e @ v[:, h]) / (e.sum(-1, keepdim=True) + torch.exp(w[p + "sink"][h] - top))
    return out.reshape(n, heads * vdim) @ w[p + "o"].T


def polynorm(z, coef, eps):
    a, b, c, e = coef
    return a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e


def dense_ffn(w, p, a, eps):
    return polynorm(a @ w[p + "up"].T, w[p + "act"], eps) @ w[p + "down"].T


def expert(w, p, a):
    gate = a @ w[p + "gate"].T
    return (gate * torch.sigmoid(gate) * (a @ w[p + "up"].T)) @ w[p + "down"].T


def choose(scores, correction, router):
    """scores [E] -> the indices of the chosen experts."""
    choice = scores + correction
    experts = scores.shape[0]
    allowed = torch.ones(experts, dtype=torch.bool)
    groups = router.get("groups")
    if groups:
        size = experts // groups["count"]
        of_group = [choice[g * size: (g + 1) * size].sort(descending=True).values[:2].sum() for g in range(groups["count"])]
        best = sorted(range(groups["count"]), key=lambda g: -float(of_group[g]))[: groups["keep"]]
        allowed = torch.tensor([e // size in best for e in range(experts)])
    ranked = sorted((e for e in range(experts) if allowed[e]), key=lambda e: -float(choice[e]))
    return ranked[: router["top"]]


def moe_ffn(w, p, mlp, a):
    router = mlp["router"]
    scores = torch.sigmoid(a @ w[p + "router"].T)
    out = torch.zeros_like(a)
    for t in range(a.shape[0]):
        for e in choose(scores[t], w[p + "correction"], router):
            out[t] += router["scale"] * scores[t, e] * expert(w, f"{p}e{e}.", a[t: t + 1])[0]
    if mlp.get("shared"):
        out = out + expert(w, p + "shared.", a)
    return out


def run_order(config):
    """[(layer, pass number or None)]: the pass number where a pass of the loop begins."""
    n, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def forward(config, tensors, ids, dtype=torch.float64):
    """-> (logits [n, vocab], the residual stream after every layer run [[n, W]])."""
    w = {k: v.to(dtype) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(ids)] * config.get("embedding", {}).get("scale", 1.0)
    streams = []
    for i, begins in run_order(config):
        layer, p = config["layers"][i], f"l{i}."
        if begins is not None:
            x = x + w["loop.step"][begins]
        a = rms(x, eps) * w[p + "norm1"]
        if config.get("canon"):
            a = causal_filter(a, w[p + "canon1"])
        mixer = attention if layer["type"] == "attention" else latent_attention
        y = mixer(w, p + "mix.", layer["mixer"], a, eps)
        mlp = layer.get("mlp")
        if mlp:
            b = rms(x, eps) * w[p + "norm2"]
            if config.get("canon"):
                b = causal_filter(b, w[p + "canon2"])
            y = y + (dense_ffn(w, p + "mlp.", b, eps) if mlp["kind"] == "dense" else moe_ffn(w, p + "mlp.", mlp, b))
        x = x + y
        streams.append(x)
    return (rms(x, eps) * w["final.norm"]) @ w["head"].T, streams
