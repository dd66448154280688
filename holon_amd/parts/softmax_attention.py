"""Softmax attention over the paged cache for heads whose keys and values may differ in width, with the options a
design may name: biases on the q/k/v projections, rotary positions in either pairing, a scale of its own, a sliding
window (which may keep the first tokens of the sequence visible), a sink (one trained scalar for each head whose
exponential is added to the softmax's normaliser; nothing is read from the cache for it), one RMS norm over a token's
whole query or key projection, a tanh cap on the scores and a logarithmic distance bias per head.
Two mixers use it: `attention` (grouped queries) and `latent_attention` (keys and values rebuilt from a cached
low-rank latent, computed in the latent's space so that nothing but the latent is kept).

Pages are laid out as the sigmoid attention lays them out (`parts/sigmoid_attention.py`): keys `[Hkv, P, D]`, then
values `[Hkv, V, P]`; `head_prepare` writes them. HIP form: `csrc/softmax_attention.hip`.
"""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import FLOAT32, Build, PagedState, Part
from .linear import Linear

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return None if t is None else t.data_ptr()


def softmax_attention_plain(q, pages, table, rows, token_row, positions, kv_heads, vdim, page_size, sink, scale,
                            window, softcap=0.0, dist=None, keep_first=0, value_share=1):
    """q [T, H, D]; `pages` [pages, G P (D + V)] (keys [G, P, D], then values [G, V, P]); `table` [S, max_pages]
    int32; token t belongs to row token_row[t] (slot rows.slots[row]) and stands at positions[t]. Query at position p
    sees keys max(0, p - window + 1) .. p (window 0: 0 .. p). weights = exp(s_j - top) / (sum_j exp(s_j - top) +
    exp(sink[h] - top)) with s = q . k * scale, `sink` [H] float32 or None (then no such term). With a window and
    `keep_first` > 0 the query also sees keys 0 .. keep_first - 1, at their true positions. `softcap` > 0: s <-
    softcap tanh(s / softcap); `dist` = (r1 [H], r2 [H]) float32: then s <- s - r1 ln(1 + r2 (p - j)) for the key at
    position j. `value_share` s > 1: a page holds G / s value heads behind its G key heads, and key head g reads value
    head g // s. -> [T, H V] in q's dtype; scores, weights and sums in float32."""
    t, heads, dim = q.shape
    keys = pages[:, : kv_heads * page_size * dim].view(-1, kv_heads, page_size, dim)
    vals = pages[:, kv_heads * page_size * dim:].view(-1, kv_heads // value_share, vdim, page_size).transpose(2, 3)
    if value_share > 1:
        vals = vals.repeat_interleave(value_share, dim=1)
    out = torch.zeros((t, heads, vdim), dtype=torch.float32, device=q.device)
    pos = positions.tolist()
    slot_of, row_of = rows.slots.tolist(), token_row.tolist()
    group = heads // kv_heads
    for i in range(t):
        first = max(0, pos[i] - window + 1) if window > 0 else 0
        js = torch.arange(first, pos[i] + 1, device=q.device)
        if keep_first > 0 and first > 0:
            js = torch.cat((torch.arange(0, min(keep_first, first), device=q.device), js))
        pg = table[slot_of[row_of[i]], (js // page_size)].long()
        off = js % page_size
        kk = keys[pg, :, off].float().repeat_interleave(group, dim=1)                  # [n, H, D]
        vv = vals[pg, :, off].float().repeat_interleave(group, dim=1)                  # [n, H, V]
        s = torch.einsum("hd,nhd->nh", q[i].float(), kk) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if dist is not None:
            s = s - dist[0].float() * torch.log1p(dist[1].float() * (pos[i] - js).float()[:, None])
        top = s.max(0).values
        if sink is not None:
            top = torch.maximum(top, sink.float())
        w = torch.exp(s - top)
        den = w.sum(0)
        if sink is not None:
            den = den + torch.exp(sink.float() - top)
        out[i] = torch.einsum("nh,nhv->hv", w, vv) / den[:, None]
    return out.view(t, heads * vdim).to(q.dtype)


def _softmax_attention_hip(launch, q, pages, table, rows, token_row, positions, kv_heads, vdim, page_size, sink,
                           scale, window, softcap=0.0, dist=None, keep_first=0, value_share=1):
    t, heads, dim = q.shape
    if dist is not None and not all(d.is_cuda and d.dtype == torch.float32 and d.is_contiguous() and d.shape == (heads,)
                                    for d in dist):
        raise ValueError("softmax_attention: the distance bias is two float32 numbers a head")
    ok = q.is_cuda and q.is_contiguous() and q.dtype in _DT and pages.dtype == q.dtype and pages.is_contiguous() \
        and pages.dim() == 2 and value_share >= 1 and kv_heads % value_share == 0 \
        and pages.shape[1] == kv_heads * page_size * dim + kv_heads // value_share * page_size * vdim \
        and table.dtype == torch.int32 \
        and table.is_contiguous() and heads % kv_heads == 0 and token_row.shape[0] >= t and positions.shape[0] >= t \
        and (sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.shape == (heads,)))
    if not ok:
        raise ValueError(f"softmax_attention: q {tuple(q.shape)} {q.dtype}, pages {tuple(pages.shape)} do not fit "
                         f"{kv_heads} kv heads, values of {vdim}, page {page_size}")
    out = torch.empty((t, heads * vdim), dtype=q.dtype, device=q.device)
    launch(q.data_ptr(), out.data_ptr(), pages.data_ptr(), table.data_ptr(), table.shape[1], table.shape[0],
           rows.slots.data_ptr(), token_row.data_ptr(), positions.data_ptr(), t, heads, kv_heads, dim, vdim, page_size,
           pages.shape[0], _ptr(sink), float(scale), int(window), _DT[q.dtype], float(softcap),
           _ptr(dist[0]) if dist is not None else None, _ptr(dist[1]) if dist is not None else None, int(keep_first),
           int(value_share))
    return out


def head_linear_plain(x, weight, out=None):
    """x [T, H, A], weight [H, B, A] -> [T, H, B]: every head's own small projection, sums in float32, the result in
    x's dtype. `out`: where the result goes, the first B columns of every head of a tensor [T, H, B'] with B' >= B
    (a view whose last dimension is contiguous); it is returned."""
    y = torch.einsum("tha,hba->thb", x, weight.to(x.dtype))
    if out is None:
        return y.contiguous()
    out.copy_(y)
    return out


def _head_linear_hip(launch, x, weight, out=None):
    """Steps of up to 16 rows: this package's kernel (the weights stream once, no copy of the result); more rows: the
    vendor library's batched product."""
    t, heads, a = x.shape
    b = weight.shape[1]
    if not (x.is_cuda and x.is_contiguous() and weight.is_contiguous() and weight.dtype == x.dtype and x.dtype in _DT
            and tuple(weight.shape) == (heads, b, a)):
        raise ValueError(f"head_linear: rows {tuple(x.shape)} {x.dtype} do not fit weights {tuple(weight.shape)} {weight.dtype}")
    if out is not None and not (out.shape == (t, heads, b) and out.dtype == x.dtype and out.stride(2) == 1
                                and out.stride(0) == heads * out.stride(1) and out.stride(1) >= b):
        raise ValueError(f"head_linear: the result's place {tuple(out.shape)} with strides {out.stride()} does not fit")
    if not 1 <= t <= 16 or t * a * 4 > 48 * 1024:
        return head_linear_plain(x, weight, out)
    y = out if out is not None else torch.empty((t, heads, b), dtype=x.dtype, device=x.device)
    launch(x.data_ptr(), weight.data_ptr(), y.data_ptr(), t, heads, a, b, y.stride(1), _DT[x.dtype])
    return y


def whole_norm_prepare_plain(qkv, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, pages, write_page, write_off,
                             page_size):
    """qkv [T, H D + G D + G V] (the merged projection). The H D query values of a token are divided by their root
    mean square as one vector (eps inside the root) and multiplied by `q_weight` [H D]; the G D key values likewise
    with `k_weight`; float32 inside, one rounding. The keys and the values go into `pages` [pages, G P (D + V)] (keys
    [G, P, D], then values [G, V, P]) at (write_page[t], write_off[t]); returns the queries [T, H, D]."""
    t = qkv.shape[0]
    nq, nk = heads * dim, kv_heads * dim

    def norm(x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(qkv.dtype)
    q = norm(qkv[:, :nq], q_weight).view(t, heads, dim)
    k = norm(qkv[:, nq: nq + nk], k_weight).view(t, kv_heads, dim)
    v = qkv[:, nq + nk:].view(t, kv_heads, vdim)
    keys = pages[:, : kv_heads * page_size * dim].view(-1, kv_heads, page_size, dim)
    vals = pages[:, kv_heads * page_size * dim:].view(-1, kv_heads, vdim, page_size)
    keys[write_page.long(), :, write_off.long()] = k
    vals[write_page.long(), :, :, write_off.long()] = v
    return q.contiguous()


def _whole_norm_prepare_hip(launch, qkv, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, pages, write_page,
                            write_off, page_size):
    t = qkv.shape[0]
    ok = qkv.is_cuda and qkv.is_contiguous() and qkv.dtype in _DT and qkv.shape[1] == (heads + kv_heads) * dim + kv_heads * vdim \
        and pages.dtype == qkv.dtype and pages.is_contiguous() and pages.dim() == 2 \
        and pages.shape[1] == kv_heads * page_size * (dim + vdim) \
        and q_weight.dtype == qkv.dtype and k_weight.dtype == qkv.dtype and q_weight.is_contiguous() \
        and k_weight.is_contiguous() and q_weight.shape == (heads * dim,) and k_weight.shape == (kv_heads * dim,) \
        and write_page.shape[0] >= t and write_off.shape[0] >= t
    if not ok:
        raise ValueError(f"whole_norm_prepare: rows {tuple(qkv.shape)} {qkv.dtype}, pages {tuple(pages.shape)} do not fit "
                         f"{heads}/{kv_heads} heads of {dim}/{vdim}, page {page_size}")
    q = torch.empty((t, heads, dim), dtype=qkv.dtype, device=qkv.device)
    if t:
        launch(qkv.data_ptr(), t, heads, kv_heads, dim, vdim, q_weight.data_ptr(), k_weight.data_ptr(), float(eps),
               q.data_ptr(), pages.data_ptr(), write_page.data_ptr(), write_off.data_ptr(), page_size, pages.shape[0],
               _DT[qkv.dtype])
    return q


def latent_rope_prepare_plain(both, heads, dim, rot, kv_rank, c_weight, eps, table, positions, pages, write_page,
                              write_off, page_size):
    """both [T, H (dim + rot) + kv_rank + rot]: every head's query as [dim unrotated, rot rotated], then the latent's
    projection and one rotated key part that all heads share. The latent is divided by its root mean square and
    multiplied by `c_weight` (float32 inside, one rounding); the first table.shape[1] dimensions of every rotated part
    (queries and key) are rotated by the token's position, half-split pairing, `table` [positions, rotary_dim] float32
    holding cosines then sines. The token's cache entry [latent, rotated key part] goes into `pages` [pages, 2 P
    (kv_rank + rot)] twice, as a key (row of [P, kv_rank + rot]) and as a value (column of [kv_rank + rot, P]).
    Returns (the unrotated query parts [T, H, dim], the queries in the cache's space [T, H, kv_rank + rot] with the
    rotated parts in their last `rot` columns and the first kv_rank left for the caller to fill)."""
    t = both.shape[0]
    width = kv_rank + rot
    q = both[:, : heads * (dim + rot)].view(t, heads, dim + rot)
    tail = both[:, heads * (dim + rot):]
    cf = tail[:, :kv_rank].float()
    c = (cf * torch.rsqrt(cf.pow(2).mean(-1, keepdim=True) + eps) * c_weight.float()).to(both.dtype)
    rd = table.shape[1] if table is not None else 0

    def turn(x):                                   # x [T, n, rot]
        if not rd:
            return x
        cs = table[positions[:t].long()]
        cos, sin = cs[:, None, : rd // 2], cs[:, None, rd // 2:]
        a, b = x[..., : rd // 2].float(), x[..., rd // 2: rd].float()
        return torch.cat(((a * cos - b * sin).to(x.dtype), (b * cos + a * sin).to(x.dtype), x[..., rd:]), dim=-1)
    entry = torch.cat((c, turn(tail[:, None, kv_rank:])[:, 0]), dim=-1)
    keys = pages[:, : page_size * width].view(-1, page_size, width)
    vals = pages[:, page_size * width:].view(-1, width, page_size)
    keys[write_page[:t].long(), write_off[:t].long()] = entry
    vals[write_page[:t].long(), :, write_off[:t].long()] = entry
    full = torch.zeros((t, heads, width), dtype=both.dtype, device=both.device)
    full[..., kv_rank:] = turn(q[..., dim:])
    return q[..., :dim].contiguous(), full


def _latent_rope_prepare_hip(launch, both, heads, dim, rot, kv_rank, c_weight, eps, table, positions, pages, write_page,
                             write_off, page_size):
    t = both.shape[0]
    width = kv_rank + rot
    rd = table.shape[1] if table is not None else 0
    ok = both.is_cuda and both.is_contiguous() and both.dtype in _DT and both.shape[1] == heads * (dim + rot) + width \
        and pages.dtype == both.dtype and pages.is_contiguous() and pages.dim() == 2 \
        and pages.shape[1] == 2 * page_size * width and c_weight.dtype == both.dtype and c_weight.is_contiguous() \
        and c_weight.shape == (kv_rank,) and write_page.shape[0] >= t and write_off.shape[0] >= t \
        and positions.shape[0] >= t and rd % 2 == 0 and rd <= rot \
        and (table is None or (table.dtype == torch.float32 and table.is_contiguous()))
    if not ok:
        raise ValueError(f"latent_rope_prepare: rows {tuple(both.shape)} {both.dtype}, pages {tuple(pages.shape)} do not "
                         f"fit {heads} heads of {dim} + {rot}, a latent of {kv_rank}, page {page_size}")
    q = torch.empty((t, heads, dim), dtype=both.dtype, device=both.device)
    full = torch.empty((t, heads, width), dtype=both.dtype, device=both.device)
    if t:
        launch(both.data_ptr(), t, heads, dim, rot, kv_rank, c_weight.data_ptr(), float(eps), _ptr(table), rd,
               table.shape[0] if table is not None else 0, positions.data_ptr(), q.data_ptr(), full.data_ptr(),
               pages.data_ptr(), write_page.data_ptr(), write_off.data_ptr(), page_size, pages.shape[0], _DT[both.dtype])
    return q, full


def latent_prepare_plain(both, q_rank, q_weight, c_weight, eps, pages, write_page, write_off, page_size):
    """both [T, q_rank + R] (the two latents' projections side by side): each x * rsqrt(mean(x^2) + eps) * weight,
    float32 inside, one rounding. Returns the first [T, q_rank]; the second goes into `pages` [pages, 2 P R] at
    (write_page[t], write_off[t]) twice: as a key (row of [P, R]) and as a value (column of [R, P])."""
    t, rank = both.shape[0], both.shape[1] - q_rank

    def norm(x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(both.dtype)
    cq, c = norm(both[:, :q_rank], q_weight), norm(both[:, q_rank:], c_weight)
    keys = pages[:, : page_size * rank].view(-1, page_size, rank)
    vals = pages[:, page_size * rank:].view(-1, rank, page_size)
    keys[write_page.long(), write_off.long()] = c
    vals[write_page.long(), :, write_off.long()] = c
    return cq.contiguous()


def _latent_prepare_hip(launch, both, q_rank, q_weight, c_weight, eps, pages, write_page, write_off, page_size):
    t, rank = both.shape[0], both.shape[1] - q_rank
    ok = both.is_cuda and both.is_contiguous() and both.dtype in _DT and rank > 0 and pages.dtype == both.dtype \
        and pages.is_contiguous() and pages.dim() == 2 and pages.shape[1] == 2 * page_size * rank \
        and all(w.dtype == both.dtype and w.is_contiguous() for w in (q_weight, c_weight)) \
        and q_weight.shape == (q_rank,) and c_weight.shape == (rank,) and write_page.shape[0] >= t \
        and write_off.shape[0] >= t
    if not ok:
        raise ValueError(f"latent_prepare: rows {tuple(both.shape)} {both.dtype}, pages {tuple(pages.shape)} do not fit "
                         f"latents of {q_rank} and {rank}, page {page_size}")
    cq = torch.empty((t, q_rank), dtype=both.dtype, device=both.device)
    launch(both.data_ptr(), t, q_rank, rank, q_weight.data_ptr(), c_weight.data_ptr(), float(eps), cq.data_ptr(),
           pages.data_ptr(), write_page.data_ptr(), write_off.data_ptr(), page_size, pages.shape[0], _DT[both.dtype])
    return cq


def head_gate_plain(x, gates, heads):
    """x [T, H V], updated in place: head h of token t is multiplied by sigmoid(gates[t, h]); `gates` [T, H] may be
    columns of wider rows (a view with a row stride). float32 inside, one rounding."""
    t = x.shape[0]
    v = x.view(t, heads, -1)
    v.copy_((v.float() * torch.sigmoid(gates.float())[:, :, None]).to(x.dtype))
    return x


def _head_gate_hip(launch, x, gates, heads):
    t = x.shape[0]
    if not (x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.dtype in _DT and x.shape[1] % heads == 0
            and gates.dtype == x.dtype and gates.shape == (t, heads) and gates.stride(1) == 1):
        raise ValueError(f"head_gate: rows {tuple(x.shape)} {x.dtype} and gates {tuple(gates.shape)} {gates.dtype} "
                         f"(strides {gates.stride()}) do not fit {heads} heads")
    if t:
        launch(x.data_ptr(), gates.data_ptr(), gates.stride(0), t, heads, x.shape[1] // heads, _DT[x.dtype])
    return x


def add_bias_plain(x, bias):
    """x [T, N] += bias [N] (float32) in place: the sum in float32, one rounding."""
    x.copy_((x.float() + bias.float()).to(x.dtype))
    return x


def _add_bias_hip(launch, x, bias):
    if not (x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.dtype in _DT and bias.is_contiguous()
            and bias.dtype == torch.float32 and bias.shape == (x.shape[1],)):
        raise ValueError(f"add_bias: rows {tuple(x.shape)} {x.dtype} and a bias {tuple(bias.shape)} {bias.dtype}")
    if x.shape[0]:
        launch(x.data_ptr(), bias.data_ptr(), x.shape[0], x.shape[1], _DT[x.dtype])
    return x


register_kernel(KernelOp("softmax_attention", softmax_attention_plain, "holon_softmax_attention",
                         [_P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _F, _I, _I, _F, _P, _P, _I, _I],
                         _softmax_attention_hip))
register_kernel(KernelOp("head_linear", head_linear_plain, "holon_head_linear_rows",
                         [_P, _P, _P, _I, _I, _I, _I, _I, _I], _head_linear_hip))
register_kernel(KernelOp("whole_norm_prepare", whole_norm_prepare_plain, "holon_whole_norm_prepare",
                         [_P, _I, _I, _I, _I, _I, _P, _P, _F, _P, _P, _P, _P, _I, _I, _I], _whole_norm_prepare_hip))
register_kernel(KernelOp("latent_rope_prepare", latent_rope_prepare_plain, "holon_latent_rope_prepare",
                         [_P, _I, _I, _I, _I, _I, _P, _F, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I],
                         _latent_rope_prepare_hip))
register_kernel(KernelOp("latent_prepare", latent_prepare_plain, "holon_latent_prepare",
                         [_P, _I, _I, _I, _P, _P, _F, _P, _P, _P, _P, _I, _I, _I], _latent_prepare_hip))
register_kernel(KernelOp("head_gate", head_gate_plain, "holon_head_gate", [_P, _P, _L, _L, _I, _I, _I], _head_gate_hip))
register_kernel(KernelOp("add_bias", add_bias_plain, "holon_add_bias", [_P, _P, _L, _I, _I], _add_bias_hip))


def attend(k, q, held, view, step, kv_heads, vdim, sink, scale, window, softcap=0.0, dist=None, keep_first=0,
           value_share=1, head_gate=None):
    """The attention of the mixers: on the matrix cores where keys and values have one width that those kernels
    serve (the pages' layout is then theirs), else the general kernel. q [T, H, D] -> [T, H V]. `value_share` s > 1:
    a page holds kv_heads / s value heads behind its kv_heads key heads, and key head g reads value head g // s.
    `head_gate` [T, H] (a view with a row stride will do): head h's result is multiplied by sigmoid(head_gate[t, h]),
    in the matrix-core kernels' last step, else by a kernel of its own behind the general one."""
    t, heads, dim = q.shape
    keep = keep_first if window > 0 else 0
    more = {} if head_gate is None else {"head_gate": head_gate}       # (only named where there is one)
    if dim == vdim and k.attention_on_cores(dim, view.page_size, q.dtype):
        if value_share > 1:
            pages = held.pages.view(-1, kv_heads + kv_heads // value_share, view.page_size * dim)
            return k.paged_attention(q, pages, view.table, step.rows, view.page_size, scale, window, sink=sink,
                                     softcap=softcap, dist=dist, keep_first=keep, value_share=value_share, **more
                                     ).view(t, heads * vdim)
        pages = held.pages.view(-1, 2, kv_heads, view.page_size * dim)
        return k.paged_attention(q, pages, view.table, step.rows, view.page_size, scale, window, sink=sink,
                                 softcap=softcap, dist=dist, keep_first=keep, **more).view(t, heads * vdim)
    if value_share > 1:
        out = k.softmax_attention(q, held.pages, view.table, step.rows, step.token_row, step.positions, kv_heads, vdim,
                                  view.page_size, sink, scale, window, softcap=softcap, dist=dist, keep_first=keep,
                                  value_share=value_share)
    else:
        out = k.softmax_attention(q, held.pages, view.table, step.rows, step.token_row, step.positions, kv_heads, vdim,
                                  view.page_size, sink, scale, window, softcap=softcap, dist=dist, keep_first=keep)
    return out if head_gate is None else k.head_gate(out, head_gate, heads)


def to_half_split(rows_per_head: int, heads: int, rot: int) -> torch.Tensor:
    """The order of a projection's output rows that turns the interleaved pairing of rotary dimensions, (2i, 2i + 1),
    into the half-split one, (i, i + rot/2), head by head; rows from `rot` on stay. Queries and keys permuted alike
    keep every score."""
    one = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, rows_per_head))
    return torch.tensor([h * rows_per_head + r for h in range(heads) for r in one], dtype=torch.long)


@register_part("mixer", "attention")
class SoftmaxAttention(Part):
    """Grouped-query softmax attention: q/k/v projections (one merged product) with optional biases (`qkv_bias`),
    optional rotary positions (`position`: any registered position part with a `table`; one that says `interleaved`
    has its pairing turned into the kernels' by reordering the projections' rows once), `scale`, an optional window
    and an optional sink per head (`sink`), output projection. Keys are `dim` wide, values `vdim`.

    Further options: `whole_norm` (an eps): all of a token's query values are RMS-normed as one vector before they
    are split into heads, with a weight `q_norm` of that length, and its key values likewise (`k_norm`); `softcap`:
    scores become softcap tanh(score / softcap); `distance_bias`: r1_h ln(1 + r2_h (i - j)) is taken off the score of
    key j for query i (`r1`, `r2`, one number a head each); `keep_first`: under a window the first tokens of the
    sequence stay visible, at their true positions.

    `values_from_keys`: there is no value projection; a token's values are its keys straight from the projection (bias added, before
    the rotation), so vdim = dim, and the cache holds the turned key and the unturned one side by side. `sink_value`
    (a number): a sink that every head shares and no tensor holds (0: one is added to the softmax's denominator).
    `head_gate`: a projection `g` of one number a head, computed with q and k in the merged product; head h's result
    is multiplied by sigmoid(g_h) before the output projection. `o_bias`: a bias on the output projection."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, kv_heads: int, dim: int, vdim: int, hidden: int, layer: int,
                 scale: float | None = None, window: int = 0, qkv_bias: bool = False, sink: bool = False,
                 position: PartRef | None = None, name: str = "", whole_norm: float | None = None,
                 softcap: float = 0.0, distance_bias: bool = False, keep_first: int = 0,
                 values_from_keys: bool = False, sink_value: float | None = None, head_gate: bool = False,
                 o_bias: bool = False) -> None:
        super().__init__(build)
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} heads are not a multiple of {kv_heads} kv heads")
        self.values_from_keys = bool(values_from_keys)
        if self.values_from_keys and vdim != dim:
            raise ValueError(f"attention: values that are the keys are as wide as the keys ({dim}), not {vdim}")
        if self.values_from_keys and whole_norm is not None:
            raise ValueError("attention: values from the keys come without the norm over the whole projection")
        if sink and sink_value is not None:
            raise ValueError("attention: either a sink per head or one number for all")
        if head_gate and whole_norm is not None:
            raise ValueError("attention: the gate per head comes without the norm over the whole projection")
        self.heads, self.kv_heads, self.dim, self.vdim, self.hidden = heads, kv_heads, dim, vdim, hidden
        self.window = int(window)
        self.keep_first = int(keep_first) if self.window > 0 else 0
        self.softcap = float(softcap or 0.0)
        self.whole_norm = None if whole_norm is None else float(whole_norm)
        if self.whole_norm is not None:
            if qkv_bias or position is not None:
                raise ValueError("attention: the norm over the whole projection comes without biases and rotation")
            self.declare("q_norm", (heads * dim,), init="norm")
            self.declare("k_norm", (kv_heads * dim,), init="norm")
        self.distance_bias = bool(distance_bias)
        if self.distance_bias:
            self.declare("r1", (heads,), kind=FLOAT32, init="unit")
            self.declare("r2", (heads,), kind=FLOAT32, init="unit")
        self.scale = float(scale) if scale is not None else dim ** -0.5
        self.state_name = f"{name}.kv" if name else "kv"
        self.attach("q", Linear(build, inp=hidden, out=heads * dim))
        self.attach("k", Linear(build, inp=hidden, out=kv_heads * dim))
        if not self.values_from_keys:
            self.attach("v", Linear(build, inp=hidden, out=kv_heads * vdim))
        self.has_gate = bool(head_gate)
        if self.has_gate:
            self.attach("g", Linear(build, inp=hidden, out=heads))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.qkv_bias = bool(qkv_bias)
        if self.qkv_bias:
            self.declare("q_bias", (heads * dim,), kind=FLOAT32, init="zero")
            self.declare("k_bias", (kv_heads * dim,), kind=FLOAT32, init="zero")
            if not self.values_from_keys:
                self.declare("v_bias", (kv_heads * vdim,), kind=FLOAT32, init="zero")
        self.has_o_bias = bool(o_bias)
        if self.has_o_bias:
            self.declare("o_bias", (hidden,), kind=FLOAT32, init="zero")
        self.has_sink = bool(sink)
        if self.has_sink:
            self.declare("sink", (heads,), kind=FLOAT32, init="zero")
        self.sink_value = None if sink_value is None else float(sink_value)
        self.position = None
        if position is not None:
            self.attach("position", build.make(position, head_dim=dim))
        self.qkv: Linear | None = None
        self.bias: torch.Tensor | None = None
        self.fixed_sink: torch.Tensor | None = None
        self.qkv_width = (heads + kv_heads) * dim + (0 if self.values_from_keys else kv_heads * vdim)

    def state(self):
        return [PagedState(self.state_name, elems=self.kv_heads * (self.dim + self.vdim), window=self.window,
                           keep_first=self.keep_first)]

    def finalize(self) -> None:
        if self.q.weight is not None and getattr(self.position, "interleaved", False):
            rot = self.position.rotary_dim
            for proj, heads, bias in ((self.q, self.heads, "q_bias"), (self.k, self.kv_heads, "k_bias")):
                order = to_half_split(self.dim, heads, rot).to(proj.weight.device)
                proj.weight = proj.weight.index_select(0, order).contiguous()
                if self.qkv_bias:
                    setattr(self, bias, getattr(self, bias).index_select(0, order).contiguous())
        if self.qkv_bias and self.q_bias is not None:
            self.bias = torch.cat([self.q_bias, self.k_bias] + ([] if self.values_from_keys else [self.v_bias])
                                  ).contiguous()
        if self.sink_value is not None and self.build.device.type != "meta":
            self.fixed_sink = torch.full((self.heads,), self.sink_value, dtype=torch.float32, device=self.build.device)
        merged = ["q", "k"] + ([] if self.values_from_keys else ["v"]) + (["g"] if self.has_gate else [])
        if self.has_gate and self.g.weight is not None and self.heads % 16:
            # the gates' columns are padded with rows of zeros to a multiple of 16: every product of the framework
            # then serves the merged projection
            pad = 16 - self.heads % 16
            self.g.weight = torch.cat((self.g.weight, self.g.weight.new_zeros((pad, self.hidden)))).contiguous()
            self.g.out += pad
        self.qkv = Linear.merge(self.build, *(getattr(self, name) for name in merged))
        for name in merged:
            self.drop(name)
        self._children["qkv"] = self.qkv

    def extra_tensors(self):
        return [t for t in (self.bias, self.fixed_sink) if t is not None]

    @property
    def out_row(self) -> torch.Tensor | None:
        """The output projection's bias, for a caller that adds it to the stream itself (`forward(add_row=False)`)."""
        return self.o_bias if self.has_o_bias else None

    def forward(self, x: torch.Tensor, step, site, add_row: bool = True) -> torch.Tensor:
        k = self.kernels
        held = site.paged[self.state_name]
        view = step.paged[held.group]
        table = getattr(self.position, "table", None)
        qkv = self.qkv(x)
        if self.whole_norm is not None:
            q = k.whole_norm_prepare(qkv, self.heads, self.kv_heads, self.dim, self.vdim, self.q_norm,
                                     self.k_norm, self.whole_norm, held.pages, view.write_page, view.write_off,
                                     view.page_size)
        else:
            q = k.head_prepare(qkv, self.heads, self.kv_heads, self.dim, self.vdim, None, None, 0.0, table,
                               step.positions, held.pages, view.write_page, view.write_off, view.page_size,
                               bias=self.bias, values="keys" if self.values_from_keys else "own")
        sink = self.sink if self.has_sink else self.fixed_sink
        gates = qkv[:, self.qkv_width: self.qkv_width + self.heads] if self.has_gate else None
        out = attend(k, q, held, view, step, self.kv_heads, self.vdim, sink, self.scale,
                     self.window, self.softcap, (self.r1, self.r2) if self.distance_bias else None, self.keep_first,
                     head_gate=gates)
        out = self.o(out)
        return k.add_bias(out, self.o_bias) if self.has_o_bias and add_row else out

    __call__ = forward


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    """Attention whose keys and values are rebuilt from a cached low-rank latent:

        c = norm(W_dkv x),  k_h = W_uk,h c,  v_h = W_uv,h c

    Only c [kv_rank] is cached per token. The scores q_h . k_h equal (W_uk,h^T q_h) . c, and the weighted sum of the
    v_h equals W_uv,h applied to the weighted sum of the c: the mixer attends in the latent's space, with one shared
    key/value head whose keys and values are both c, and applies W_uk,h to the queries and W_uv,h to the results, head
    by head. `norm` is the kind of the latents' norms (their `eps` comes with it); `window` 0 sees everything before.

    Two forms of the queries. `q_rank` > 0: through a latent of their own, c_q = norm(W_dq x), q_h = W_uq,h c_q, no
    positions. `q_rank` 0: q = W_q x, every head laid out as [dim unrotated, rot_dim rotated], and W_dkv has rot_dim
    more rows, one rotated key part that all heads share (not normed); the score is the sum of the unrotated and the
    rotated products. The cache entry is then [c, rotated key part], kept as key and as value (W_uv,h gets zero
    columns for the rotated part). `position` (a registered position part with a `table`) rotates the first
    `rotary_dim` of the rot_dim dimensions; one that says `interleaved` has the rows of W_q and W_dkv reordered once
    so that the kernels' half-split pairing rotates the design's pairs. `sink`: one number a head in the softmax's
    denominator."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, dim: int, vdim: int, kv_rank: int, norm: PartRef, hidden: int,
                 layer: int, q_rank: int = 0, rot_dim: int = 0, position: PartRef | None = None, sink: bool = False,
                 scale: float | None = None, window: int = 0, name: str = "") -> None:
        super().__init__(build)
        if q_rank > 0 and (rot_dim > 0 or position is not None):
            raise ValueError("latent_attention: queries through a latent of their own come without a rotated part")
        if position is not None and rot_dim < 2:
            raise ValueError("latent_attention: a position part needs rotated dimensions (rot_dim)")
        self.heads, self.dim, self.vdim, self.q_rank, self.kv_rank = heads, dim, vdim, int(q_rank), kv_rank
        self.rot_dim = int(rot_dim)
        self.width = kv_rank + self.rot_dim          # of a cache entry
        self.window = int(window)
        self.scale = float(scale) if scale is not None else (dim + self.rot_dim) ** -0.5
        self.state_name = f"{name}.latent" if name else "latent"
        if self.q_rank > 0:
            self.attach("dq", Linear(build, inp=hidden, out=q_rank))
            self.attach("dq_norm", build.make(norm, dim=q_rank))
            self.attach("uq", Linear(build, inp=q_rank, out=heads * dim))
        else:
            self.attach("q", Linear(build, inp=hidden, out=heads * (dim + self.rot_dim)))
        self.attach("dkv", Linear(build, inp=hidden, out=self.width))
        self.attach("dkv_norm", build.make(norm, dim=kv_rank))
        self.declare("uk", (heads * dim, kv_rank))
        self.declare("uv", (heads * vdim, kv_rank))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.has_sink = bool(sink)
        if self.has_sink:
            self.declare("sink", (heads,), kind=FLOAT32, init="zero")
        self.position = None
        if position is not None:
            self.attach("position", build.make(position, head_dim=self.rot_dim))
        self.down: Linear | None = None
        self.uk_t = self.uv_h = None
        self._fused: float | None = None          # the norms' eps, when they are RMS norms of one eps: one kernel then
                                                  # norms the latents and writes the cache

    def state(self):
        return [PagedState(self.state_name, elems=2 * self.width, window=self.window)]

    def finalize(self) -> None:
        first = self.dq if self.q_rank > 0 else self.q
        if first.weight is not None and getattr(self.position, "interleaved", False):
            rd = self.position.rotary_dim
            one = list(range(0, rd, 2)) + list(range(1, rd, 2)) + list(range(rd, self.rot_dim))
            per = self.dim + self.rot_dim
            order = [h * per + r for h in range(self.heads) for r in list(range(self.dim)) + [self.dim + r for r in one]]
            dev = first.weight.device
            self.q.weight = self.q.weight.index_select(0, torch.tensor(order, device=dev)).contiguous()
            order = list(range(self.kv_rank)) + [self.kv_rank + r for r in one]
            self.dkv.weight = self.dkv.weight.index_select(0, torch.tensor(order, device=dev)).contiguous()
        self.down = Linear.merge(self.build, first, self.dkv)
        self.drop("dq" if self.q_rank > 0 else "q")
        self.drop("dkv")
        self._children["down"] = self.down
        norms = [self.dkv_norm] + ([self.dq_norm] if self.q_rank > 0 else [])
        specs = [n.fusion() for n in norms]
        if all(sp is not None and sp.get("norm") == "rmsnorm" and sp["weight"] is not None for sp in specs) \
                and len({sp["eps"] for sp in specs}) == 1:
            self._fused = float(specs[0]["eps"])
        if self.q_rank == 0 and self._fused is None:
            raise ValueError("latent_attention: the form with a rotated part needs an RMS norm on the latent")
        if self.uk is not None:
            # [H, kv_rank, dim]: what turns a head's query into the latent's space; [H, vdim, width]: a head's values
            self.uk_t = self.uk.view(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
            self.uv_h = self.uv.view(self.heads, self.vdim, self.kv_rank)
            if self.rot_dim:
                pad = torch.zeros((self.heads, self.vdim, self.rot_dim), dtype=self.uv.dtype, device=self.uv.device)
                self.uv_h = torch.cat((self.uv_h, pad), dim=-1).contiguous()

    def extra_tensors(self):
        held = [self.uk_t] if self.uk_t is not None else []
        return held + ([self.uv_h] if self.rot_dim and self.uv_h is not None else [])

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        t = x.shape[0]
        held = site.paged[self.state_name]
        view = step.paged[held.group]
        both = self.down(x)
        if self.q_rank == 0:                      # norm, rotation and the cache write in one kernel
            q, full = k.latent_rope_prepare(both, self.heads, self.dim, self.rot_dim, self.kv_rank,
                                            self.dkv_norm.weight, self._fused, getattr(self.position, "table", None),
                                            step.positions, held.pages, view.write_page, view.write_off, view.page_size)
            k.head_linear(q, self.uk_t, out=full[..., : self.kv_rank])
            q = full
        else:
            if self._fused is not None:           # both norms and the cache write in one kernel
                cq = k.latent_prepare(both, self.q_rank, self.dq_norm.weight, self.dkv_norm.weight, self._fused,
                                      held.pages, view.write_page, view.write_off, view.page_size)
            else:
                cq = self.dq_norm(both[:, : self.q_rank].contiguous())
                c = self.dkv_norm(both[:, self.q_rank:].contiguous()).view(t, 1, self.kv_rank)
                k.kv_write(c, c, held.pages.view(-1, 2, 1, view.page_size * self.kv_rank), view.write_page,
                           view.write_off, view.page_size)
            q = k.head_linear(self.uq(cq).view(t, self.heads, self.dim), self.uk_t)
        mixed = attend(k, q, held, view, step, 1, self.width, self.sink if self.has_sink else None, self.scale,
                       self.window)
        out = k.head_linear(mixed.view(t, self.heads, self.width), self.uv_h)
        return self.o(out.view(t, self.heads * self.vdim))

    __call__ = forward
