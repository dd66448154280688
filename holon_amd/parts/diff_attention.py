"""Differential attention over the paged cache: every head attends twice, with two sets of queries and keys ("maps")
over one set of values, and its result is the first map's minus `lam` times the second's, divided by its root mean
square and multiplied by a constant:

    y_m = softmax(scale q_m k_m^T) v   (m = 1, 2; causal),   o = N(y_1 - lam y_2) gain,   N(u) = u / sqrt(mean(u^2) + eps)

The two maps are two ordinary softmax attentions, so the mixer hands the framework's attention kernels 2H query heads
over 2G key heads: the query projection's rows are reordered once after loading from (head, map) to (kv head, map, head
within the group), so that the kernels' grouping, query head // (H / G), sends map m of a head to map m of its kv
head. Key head (kv head, map) reads value head kv head: a page holds the 2G key heads and behind them the G value
heads, once, and the attention kernels are told that two key heads share a value head (`value_share=2`).
`diff_combine` puts the maps together and brings the heads back into the design's order.

Queries and keys are RMS-normed per head and map with one weight of `dim` values each (`q_norm`, `k_norm`) and turned
by a registered position part (one that says `interleaved` has the rows of both projections, and the norms' weights,
reordered so that the kernels' half-split pairing turns the design's pairs). lam is one number for the layer,
exp(lq1 . lk1) - exp(lq2 . lk2) + diff, formed once after loading in float32, and gain = 1 - diff.

`own_kv` False: the layer has no key and value projections and no key norm; its run reads the cache another run wrote
(`Run.reads`), with its own queries, lam and output projection.
"""
from __future__ import annotations

import ctypes
import math

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import FLOAT32, Build, PagedState, Part
from .linear import Linear
from .softmax_attention import attend, to_half_split

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def diff_combine_plain(y, heads, kv_heads, vdim, lam, eps, gain):
    """y [T, 2 H V]: the two maps' results, head blocks in the order (kv head, map, head within the group). ->
    [T, H V] in the order (kv head, head within the group): u = y_1 - lam y_2, then u / sqrt(mean(u^2) + eps) * gain
    over a head's V values. float32 inside, one rounding."""
    t, group = y.shape[0], heads // kv_heads
    maps = y.float().view(t, kv_heads, 2, group, vdim)
    u = maps[:, :, 0] - lam * maps[:, :, 1]
    u = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * gain
    return u.reshape(t, heads * vdim).to(y.dtype)


def _diff_combine_hip(launch, y, heads, kv_heads, vdim, lam, eps, gain):
    t = y.shape[0]
    if not (y.is_cuda and y.is_contiguous() and y.dtype in _DT and y.shape == (t, 2 * heads * vdim)
            and kv_heads > 0 and heads % kv_heads == 0):
        raise ValueError(f"diff_combine: rows {tuple(y.shape)} {y.dtype} do not hold two maps of {heads}/{kv_heads} "
                         f"heads of {vdim}")
    out = torch.empty((t, heads * vdim), dtype=y.dtype, device=y.device)
    if t:
        launch(y.data_ptr(), out.data_ptr(), t, heads, kv_heads, vdim, float(lam), float(eps), float(gain), _DT[y.dtype])
    return out


register_kernel(KernelOp("diff_combine", diff_combine_plain, "holon_diff_combine",
                         [_P, _P, _L, _I, _I, _I, _F, _F, _F, _I], _diff_combine_hip))


@register_part("mixer", "diff_attention")
class DiffAttention(Part):
    """See the module's text. `heads`, `kv_heads`: the design's counts (every one holds two maps); `dim` the width of
    a map's queries and keys, `vdim` of a head's values; `diff` the constant in lam and in the gain; `eps` the norms'."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, kv_heads: int, dim: int, vdim: int, diff: float, eps: float,
                 hidden: int, layer: int, scale: float | None = None, position: PartRef | None = None,
                 own_kv: bool = True, name: str = "") -> None:
        super().__init__(build)
        if heads % kv_heads:
            raise ValueError(f"diff_attention: {heads} heads are not a multiple of {kv_heads} kv heads")
        self.heads, self.kv_heads, self.dim, self.vdim, self.hidden = heads, kv_heads, dim, vdim, hidden
        self.diff, self.eps, self.own_kv = float(diff), float(eps), bool(own_kv)
        self.scale = float(scale) if scale is not None else dim ** -0.5
        self.state_name = f"{name}.kv" if name else "kv"
        self.attach("q", Linear(build, inp=hidden, out=2 * heads * dim))
        self.declare("q_norm", (dim,), init="norm")
        if self.own_kv:
            self.attach("k", Linear(build, inp=hidden, out=2 * kv_heads * dim))
            self.attach("v", Linear(build, inp=hidden, out=kv_heads * vdim))
            self.declare("k_norm", (dim,), init="norm")
        for name_ in ("lq1", "lk1", "lq2", "lk2"):
            self.declare(name_, (dim,), kind=FLOAT32, init="tap")
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.position = None
        if position is not None:
            self.attach("position", build.make(position, head_dim=dim))
        self.qkv: Linear | None = None
        self.lam: float | None = None

    def state(self):
        # the keys of both maps and the values, for every kv head
        return [PagedState(self.state_name, elems=self.kv_heads * (2 * self.dim + self.vdim))]

    def finalize(self) -> None:
        if self.q.weight is None:
            return
        dev = self.q.weight.device
        group = self.heads // self.kv_heads
        # query rows from (kv head, head in group, map) to (kv head, map, head in group), whole heads of `dim` rows
        blocks = [(g * group + j) * 2 + m for g in range(self.kv_heads) for m in range(2) for j in range(group)]
        order = torch.tensor([b * self.dim + r for b in blocks for r in range(self.dim)], dtype=torch.long, device=dev)
        self.q.weight = self.q.weight.index_select(0, order).contiguous()
        if getattr(self.position, "interleaved", False):
            rot = self.position.rotary_dim
            projections = [(self.q, 2 * self.heads)] + ([(self.k, 2 * self.kv_heads)] if self.own_kv else [])
            for proj, blocks_ in projections:
                order = to_half_split(self.dim, blocks_, rot).to(dev)
                proj.weight = proj.weight.index_select(0, order).contiguous()
            one = to_half_split(self.dim, 1, rot).to(dev)
            self.q_norm = self.q_norm.index_select(0, one).contiguous()
            if self.own_kv:
                self.k_norm = self.k_norm.index_select(0, one).contiguous()
        first = float((self.lq1.double() * self.lk1.double()).sum())
        second = float((self.lq2.double() * self.lk2.double()).sum())
        self.lam = float(torch.tensor(math.exp(first) - math.exp(second) + self.diff, dtype=torch.float32))
        if self.own_kv:
            self.qkv = Linear.merge(self.build, self.q, self.k, self.v)
            for name in ("q", "k", "v"):
                self.drop(name)
        else:
            self.qkv = self.q
            self.qkv.finalize()
            self.drop("q")
        self._children["qkv"] = self.qkv

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        if site.writes != self.own_kv:
            raise ValueError("diff_attention: a layer with keys and values of its own writes its cache; one without "
                             "reads another run's")
        held = site.paged[self.state_name]
        view = step.paged[held.group]
        table = getattr(self.position, "table", None)
        if self.own_kv:
            q = k.head_prepare(self.qkv(x), 2 * self.heads, 2 * self.kv_heads, self.dim, self.vdim, self.q_norm,
                               self.k_norm, self.eps, table, step.positions, held.pages, view.write_page,
                               view.write_off, view.page_size, value_share=2)
        else:
            q = k.head_prepare(self.qkv(x), 2 * self.heads, 0, self.dim, self.vdim, self.q_norm, self.q_norm,
                               self.eps, table, step.positions, None, None, None, view.page_size)
        maps = attend(k, q, held, view, step, 2 * self.kv_heads, self.vdim, None, self.scale, 0, value_share=2)
        return self.o(k.diff_combine(maps, self.heads, self.kv_heads, self.vdim, self.lam, self.eps, 1.0 - self.diff))

    __call__ = forward
