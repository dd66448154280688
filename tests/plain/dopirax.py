"""The plain Dopirax model: one function per mechanism, written from the design's equations, whole sequences at once,
no cache, no batching, float64 by default. It shares no code with the engine; the tests hold the engine to it.

Notation: x [n, W] the residual stream of a sequence of n tokens at positions 0 .. n - 1; `w` maps checkpoint tensor
names to tensors; `p` is a tensor name prefix; a = N(x) (1 + g) with N(v) = v / sqrt(mean(v^2) + eps).

  layer           x <- x + (mixer(a) + ffn(a)): one norm, read by both sublayers
  attention       q = Wq a + bq, k = Wk a + bk, v = k (from the projection, not turned); q, k turned on their first `dims`
                  dimensions in the pairing (i, i + dims / 2); s_ij = cap tanh(scale q_i . k_j / cap), j <= i;
                  p_ij = exp(s_ij) / (1 + sum_j exp(s_ij)); head h's result times sigmoid(Wg a)_h; Wo (.) + bo
  attention_2     two maps a head: q [H, 2, dim], k [G, 2, dim], v [G, vdim]; per (head, map) q <- N(q) gq, k <- N(k) gk,
                  then turned in the pairing (2i, 2i + 1); each map an ordinary causal softmax over the same values:
                  y1, y2; o = y1 - lam y2 with lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff; o <- N(o) (1 - diff); Wo.
                  With `kv_from` = j the keys (normed, turned) and values are those of layer j.
  turning         the pair (u, v) at position p becomes (u cos t - v sin t, v cos t + u sin t), t = p base^(-2i / dims)
  dense ffn       Wdown relu(Wup a)^2
  experts         z = Wr a + br; the `top` largest z are chosen, their weights softmax over the chosen z alone;
                  sum of weight_e Wdown,e (silu(Wgate,e a) * (Wup,e a)); + sigmoid(Wsg a) shared(a)
"""
from __future__ import annotations

import math

import torch


def unit(v, eps):
    return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)


def angles(n, base, dims, dtype):
    i = torch.arange(dims // 2, dtype=dtype)
    return torch.arange(n, dtype=dtype)[:, None] * base ** (-2 * i / dims)            # [n, dims / 2]


def turn_halves(u, base, dims):
    """u [n, heads, d]: dimension i paired with i + dims / 2."""
    t = angles(u.shape[0], base, dims, u.dtype)[:, None, :]
    a, b = u[..., : dims // 2], u[..., dims // 2: dims]
    return torch.cat((a * t.cos() - b * t.sin(), b * t.cos() + a * t.sin(), u[..., dims:]), dim=-1)


def turn_neighbours(u, base, dims):
    """u [n, ..., d]: dimension 2i paired with 2i + 1."""
    t = angles(u.shape[0], base, dims, u.dtype)
    t = t.view((u.shape[0],) + (1,) * (u.dim() - 2) + (dims // 2,))
    out = u.clone()
    a, b = u[..., 0:dims:2], u[..., 1:dims:2]
    out[..., 0:dims:2] = a * t.cos() - b * t.sin()
    out[..., 1:dims:2] = b * t.cos() + a * t.sin()
    return out


def hidden(n):
    return torch.arange(n)[None, :] > torch.arange(n)[:, None]


def attention(w, p, m, a, sink=True):
    n = a.shape[0]
    heads, groups, dim = m["heads"], m["kv_heads"], m["dim"]
    q = (a @ w[p + "q"].T + w[p + "q.b"]).view(n, heads, dim)
    k = (a @ w[p + "k"].T + w[p + "k.b"]).view(n, groups, dim)
    v = k
    if m.get("rot"):
        q = turn_halves(q, m["rot"]["base"], m["rot"]["dims"])
        k = turn_halves(k, m["rot"]["base"], m["rot"]["dims"])
    gate = torch.sigmoid(a @ w[p + "g"].T)                                           # [n, heads]
    out = a.new_zeros(n, heads, m["vdim"])
    for h in range(heads):
        g = h // (heads // groups)
        s = (q[:, h] @ k[:, g].T) * m["scale"]
        if m.get("softcap"):
            s = m["softcap"] * torch.tanh(s / m["softcap"])
        e = torch.exp(s).masked_fill(hidden(n), 0.0)
        out[:, h] = (e @ v[:, g]) / ((1 if sink else 0) + e.sum(-1, keepdim=True)) * gate[:, h: h + 1]
    return out.reshape(n, -1) @ w[p + "o"].T + w[p + "o.b"]


def attention_2_keys(w, p, m, a, eps):
    """The keys [n, G, 2, dim] (normed and turned) and values [n, G, vdim] that a layer of this kind makes."""
    n = a.shape[0]
    k = (a @ w[p + "k"].T).view(n, m["kv_heads"], 2, m["dim"])
    k = unit(k, eps) * w[p + "k.norm"]
    if m.get("rot"):
        k = turn_neighbours(k, m["rot"]["base"], m["rot"]["dims"])
    return k, (a @ w[p + "v"].T).view(n, m["kv_heads"], m["vdim"])


def attention_2(w, p, m, a, eps, kv):
    n = a.shape[0]
    heads, groups, dim, vdim, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["diff"]
    k, v = kv
    q = (a @ w[p + "q"].T).view(n, heads, 2, dim)
    q = unit(q, eps) * w[p + "q.norm"]
    if m.get("rot"):
        q = turn_neighbours(q, m["rot"]["base"], m["rot"]["dims"])
    lam = torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + diff
    out = a.new_zeros(n, heads, vdim)
    for h in range(heads):
        g = h // (heads // groups)
        maps = []
        for side in range(2):
            s = (q[:, h, side] @ k[:, g, side].T) * m["scale"]
            maps.append(torch.softmax(s.masked_fill(hidden(n), -math.inf), dim=-1) @ v[:, g])
        out[:, h] = unit(maps[0] - lam * maps[1], eps) * (1 - diff)
    return out.reshape(n, -1) @ w[p + "o"].T


def dense_ffn(w, p, a):
    return torch.relu(a @ w[p + "up"].T) ** 2 @ w[p + "down"].T


def expert(w, p, a):
    gate = a @ w[p + "gate"].T
    return (gate * torch.sigmoid(gate) * (a @ w[p + "up"].T)) @ w[p + "down"].T


def route(z, top):
    """z [E] -> [(expert, weight)]: the `top` largest, weighted by the softmax over them alone."""
    best = sorted(range(z.shape[0]), key=lambda e: -float(z[e]))[:top]
    weights = torch.softmax(z[best], dim=0)
    return list(zip(best, weights))


def moe_ffn(w, p, mlp, a):
    z = a @ w[p + "router"].T + w[p + "router.b"]
    out = torch.zeros_like(a)
    for t in range(a.shape[0]):
        for e, weight in route(z[t], mlp["router"]["top"]):
            out[t] += weight * expert(w, f"{p}e{e}.", a[t: t + 1])[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(a @ w[p + "shared.sg"].T) * expert(w, p + "shared.", a)
    return out


def forward(config, tensors, ids, dtype=torch.float64, sink=True):
    """-> (logits [n, vocab], the residual stream after every layer [[n, W]]). `sink` False leaves the one out of the
    attention's denominator (for tests that show what it does)."""
    w = {k: v.to(dtype) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(ids)] * config.get("embedding", {}).get("scale", 1.0)
    streams, kept = [], {}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        a = unit(x, eps) * (1 + w[p + "norm1"])
        if layer["type"] == "attention":
            y = attention(w, p + "mix.", m, a, sink)
        else:
            if m.get("kv_from") is None:
                kept[i] = attention_2_keys(w, p + "mix.", m, a, eps)
            y = attention_2(w, p + "mix.", m, a, eps, kept[m["kv_from"] if m.get("kv_from") is not None else i])
        mlp = layer.get("mlp")
        if mlp:
            y = y + (dense_ffn(w, p + "mlp.", a) if mlp["kind"] == "dense" else moe_ffn(w, p + "mlp.", mlp, a))
        x = x + y
        streams.append(x)
    return (unit(x, eps) * (1 + w["final.norm"])) @ w["head"].T, streams
