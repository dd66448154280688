"""A block whose two sublayers read the same residual stream, kept in float32:

    x += mixer(f1(norm1(x))) + ffn(f2(norm2(x)))

Both norms are RMS norms of the same rows, so they share the row's mean square and one kernel produces both results
(`stream_rms`, HIP form in `csrc/parallel_block.hip`); the same kernel first adds what the layer before left to add
(its two results, summed before they join the stream) and, for a block that opens a repeated range of layers, the
vector of the pass that begins (`pass_steps`: a tensor `[passes, hidden]` whose row `site.turn` is added in front of
every pass, the first too). f1 and f2 (`conv_taps` > 0) replace a sublayer's input a by a + conv(a), a short causal
filter over time on every channel whose last taps - 1 inputs are part of the request's state. A layer may lack the
feed-forward; its second norm and filter are then not built. With `shared_norm` the block has one norm and both
sublayers read its result: x += mixer(f1(norm1(x))) + ffn(f1(norm1(x))).

The norm `rms32` may hold its weight around zero (`one_plus`): y = x / sqrt(mean(x^2) + eps) * (1 + w); the sum 1 + w is
formed once after loading, in float32, and kept in float32 whatever the engine's dtype.
"""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import FLOAT32, Build, NormPart, Part, Stream
from .convs import CausalConv
from .stream32 import Pending, _terms

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return None if t is None else t.data_ptr()


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise ValueError(what)


def stream_rms_plain(x32, terms, row, w1, w2, eps, out_dtype):
    """x32 [T, W] float32, updated in place: x += (t1 + t2) for the `terms` [(tensor [T, W], 1.0)] (at most two, summed
    first), then x += `row` [W] float32 (None: nothing). Then r = rsqrt(mean(x^2) + eps) per row and the answers
    (x r w1, x r w2) in `out_dtype`, the second None when `w2` is; with `w1` None nothing is normed and (None, None)
    comes back. float32 arithmetic, one rounding of each answer."""
    if terms:
        add = terms[0][0].float()
        for t, _ in terms[1:]:
            add = add + t.float()
        x32.add_(add)
    if row is not None:
        x32.add_(row.float())
    if w1 is None:
        return None, None
    unit = x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)
    return (unit * w1.float()).to(out_dtype), ((unit * w2.float()).to(out_dtype) if w2 is not None else None)


def _stream_rms_hip(launch, x32, terms, row, w1, w2, eps, out_dtype):
    _need(x32.is_cuda and x32.is_contiguous() and x32.dtype == torch.float32 and x32.dim() == 2,
          "stream_rms: the stream is contiguous float32 rows on the GPU")
    _need(len(terms) <= 2 and all(float(s) == 1.0 for _, s in terms), "stream_rms: at most two terms, unscaled")
    rows, dim = x32.shape
    ptrs, dts = [None, None], [0, 0]
    for i, (term, _) in enumerate(terms):
        _need(term.is_cuda and term.is_contiguous() and term.shape == x32.shape and term.dtype in _DT,
              f"stream_rms: term {i} must be contiguous rows of the stream's shape")
        ptrs[i], dts[i] = term.data_ptr(), _DT[term.dtype]
    _need(row is None or (row.is_cuda and row.is_contiguous() and row.dtype == torch.float32 and row.shape == (dim,)),
          "stream_rms: the added row is float32 of the stream's width")
    y1 = y2 = None
    for w in (w1, w2):
        _need(w is None or (w.is_cuda and w.is_contiguous() and w.shape == (dim,) and w.dtype in _DT),
              "stream_rms: a weight of the rows' width")
    _need(w1 is not None or w2 is None, "stream_rms: a second weight without the first")
    if w1 is not None:
        _need(out_dtype in _DT, "stream_rms: float32 or bfloat16 out")
        y1 = torch.empty((rows, dim), dtype=out_dtype, device=x32.device)
        y2 = torch.empty((rows, dim), dtype=out_dtype, device=x32.device) if w2 is not None else None
    if rows:
        launch(x32.data_ptr(), ptrs[0], dts[0], ptrs[1], dts[1], _ptr(row), _ptr(w1), _ptr(w2),
               _DT[w1.dtype] if w1 is not None else 0, _ptr(y1), _ptr(y2), rows, dim, float(eps),
               _DT[out_dtype] if w1 is not None else 0)
    return y1, y2


def stream_rms_filter_plain(x32, terms, row, w1, w2, eps, out_dtype, taps1, taps2, held1, held2, slots, starts):
    """`stream_rms` for a step whose rows are single tokens (row b is token b), with each result y going through its
    causal filter, y <- y + conv(y): `taps1`, `taps2` [W, taps] and the requests' last taps - 1 inputs `held1`, `held2`
    [S, taps - 1, W] (ignored by a row that starts at 0; replaced afterwards), in `out_dtype`. The roundings are those
    of the norm and the filter one after the other."""
    from .convs import causal_conv_plain
    a, b = stream_rms_plain(x32, terms, row, w1, w2, eps, out_dtype)
    n = x32.shape[0]
    order = torch.arange(n + 1, dtype=torch.int32, device=x32.device)
    a = causal_conv_plain(a, taps1, held1, slots, starts, order, order[:n], n, True, False, True)
    if b is not None:
        b = causal_conv_plain(b, taps2, held2, slots, starts, order, order[:n], n, True, False, True)
    return a, b


def _stream_rms_filter_hip(launch, x32, terms, row, w1, w2, eps, out_dtype, taps1, taps2, held1, held2, slots, starts):
    _need(x32.is_cuda and x32.is_contiguous() and x32.dtype == torch.float32 and x32.dim() == 2,
          "stream_rms_filter: the stream is contiguous float32 rows on the GPU")
    _need(len(terms) <= 2 and all(float(s) == 1.0 for _, s in terms), "stream_rms_filter: at most two terms, unscaled")
    rows, dim = x32.shape
    taps = taps1.shape[1]
    ptrs, dts = [None, None], [0, 0]
    for i, (term, _) in enumerate(terms):
        _need(term.is_cuda and term.is_contiguous() and term.shape == x32.shape and term.dtype in _DT,
              f"stream_rms_filter: term {i} must be contiguous rows of the stream's shape")
        ptrs[i], dts[i] = term.data_ptr(), _DT[term.dtype]
    _need(row is None or (row.is_cuda and row.is_contiguous() and row.dtype == torch.float32 and row.shape == (dim,)),
          "stream_rms_filter: the added row is float32 of the stream's width")
    _need(out_dtype in _DT and w1 is not None and w1.is_contiguous() and w1.shape == (dim,) and w1.dtype in _DT
          and (w2 is None or (w2.is_contiguous() and w2.shape == (dim,) and w2.dtype == w1.dtype)),
          "stream_rms_filter: weights of the rows' width")
    for cw, held, there in ((taps1, held1, True), (taps2, held2, w2 is not None)):
        _need(not there or (cw.is_contiguous() and cw.dtype == out_dtype and cw.shape == (dim, taps)
                            and held.is_contiguous() and held.dtype == out_dtype
                            and tuple(held.shape[1:]) == (taps - 1, dim)),
              "stream_rms_filter: taps [W, taps] and held inputs [S, taps - 1, W] in the results' dtype")
    _need(slots.dtype == torch.int32 and starts.dtype == torch.int32 and slots.shape[0] >= rows and starts.shape[0] >= rows,
          "stream_rms_filter: a slot and a start for every row")
    y1 = torch.empty((rows, dim), dtype=out_dtype, device=x32.device)
    y2 = torch.empty((rows, dim), dtype=out_dtype, device=x32.device) if w2 is not None else None
    if rows:
        launch(x32.data_ptr(), ptrs[0], dts[0], ptrs[1], dts[1], _ptr(row), _ptr(w1), _ptr(w2), _DT[w1.dtype], _ptr(y1),
               _ptr(y2), rows, dim, float(eps), _DT[out_dtype], taps1.data_ptr(), _ptr(taps2) if w2 is not None else None,
               held1.data_ptr(), _ptr(held2) if w2 is not None else None, slots.data_ptr(), starts.data_ptr(), taps)
    return y1, y2


def scale_rows_plain(x, scale):
    """x [T, W] -> a new float32 tensor of scale * x."""
    return x.float() * scale


def _scale_rows_hip(launch, x, scale):
    _need(x.is_cuda and x.is_contiguous() and x.dtype in _DT, "scale_rows: contiguous float32 or bfloat16 rows on the GPU")
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    launch(x.data_ptr(), y.data_ptr(), x.numel(), _DT[x.dtype], float(scale))
    return y


register_kernel(KernelOp("stream_rms", stream_rms_plain, "holon_stream_rms",
                         [_P, _P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _L, _I, _F, _I], _stream_rms_hip))
register_kernel(KernelOp("stream_rms_filter", stream_rms_filter_plain, "holon_stream_rms_filter",
                         [_P, _P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _L, _I, _F, _I, _P, _P, _P, _P, _P, _P, _I],
                         _stream_rms_filter_hip))
register_kernel(KernelOp("scale_rows", scale_rows_plain, "holon_scale_rows", [_P, _P, _L, _I, _F], _scale_rows_hip))


@register_part("norm", "rms32")
class RMSNorm32(NormPart):
    """y = x * rsqrt(mean(x^2) + eps) * weight over rows of a float32 stream (rows in the engine's dtype are widened
    first); float32 inside, the result in the engine's dtype. `one_plus`: the stored weight w lies around zero and the
    norm multiplies by 1 + w (kept in float32: in bfloat16 the sum would lose what w holds)."""

    graph_safe = True

    def __init__(self, build: Build, *, eps: float, dim: int, one_plus: bool = False) -> None:
        super().__init__(build)
        self.eps, self.dim, self.one_plus = float(eps), dim, bool(one_plus)
        if self.one_plus:
            self.declare("weight", (dim,), kind=FLOAT32, init="tap")
        else:
            self.declare("weight", (dim,), init="norm")
        self._summed = False

    def finalize(self) -> None:
        if self.one_plus and self.weight is not None and not self._summed:
            self.weight = (self.weight.float() + 1.0).contiguous()
            self._summed = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dtype != torch.float32:
            x = self.kernels.widen_rows(x)
        return self.kernels.stream_rms(x, [], None, self.weight, None, self.eps, self.build.dtype)[0]

    __call__ = forward

    def add(self, x, residual: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """(norm(residual + x), residual + x): `residual` is float32 and takes the sum in place; `x` is a tensor or
        `Pending` terms."""
        return self.kernels.stream_rms(residual, _terms(x), getattr(x, "row", None), self.weight, None, self.eps,
                                       self.build.dtype)[0], residual

    def fusion(self) -> dict | None:
        return {"norm": "rmsnorm", "eps": self.eps, "weight": self.weight}


@register_part("block", "parallel32")
class Parallel32(Part):
    """x += mixer(f1(norm1(x))) + ffn(f2(norm2(x))) over a float32 stream; see the module's text. The norms are of
    the kind the layer names; where both are RMS norms of one eps (`fusion()`), one kernel serves both."""

    graph_safe = True

    def __init__(self, build: Build, *, layer: int, hidden: int, mixer: PartRef, ffn: PartRef | None, norm: PartRef,
                 conv_taps: int = 0, pass_steps: int = 0, shared_norm: bool = False) -> None:
        super().__init__(build)
        self.hidden = hidden
        self.shared_norm = bool(shared_norm)
        self.attach("norm1", build.make(norm, dim=hidden))
        self.attach("mixer", build.make(mixer, layer=layer, hidden=hidden))
        self.conv1 = self.conv2 = self.ffn = self.norm2 = None
        if conv_taps > 0:
            self.attach("conv1", CausalConv(build, channels=hidden, taps=conv_taps, add_input=True, name="filter1"))
        if ffn is not None:
            if not self.shared_norm:
                self.attach("norm2", build.make(norm, dim=hidden))
            self.attach("ffn", build.make(ffn, layer=layer, hidden=hidden))
            if conv_taps > 0 and not self.shared_norm:
                self.attach("conv2", CausalConv(build, channels=hidden, taps=conv_taps, add_input=True, name="filter2"))
        self.passes = int(pass_steps)
        if self.passes > 0:
            self.declare("step", (self.passes, hidden), kind=FLOAT32, init="zero")
        self._one_kernel: float | None = None      # the norms' eps when one kernel serves both
        self._fused_filter = False                 # whether a step of single tokens runs norms and filters as one kernel

    def finalize(self) -> None:
        specs = [n.fusion() for n in (self.norm1, self.norm2) if n is not None]
        if all(sp is not None and sp.get("norm") == "rmsnorm" and sp["weight"] is not None for sp in specs) \
                and len({sp["eps"] for sp in specs}) == 1:
            self._one_kernel = float(specs[0]["eps"])
            # (the kernel serves widths that are a multiple of 4 up to 8,192 and up to four taps; the plain form any)
            self._fused_filter = self.conv1 is not None and (self.ffn is None or self.conv2 is not None) \
                and not self.shared_norm \
                and self.hidden % 4 == 0 and self.hidden <= 8192 and self.conv1.taps <= 4

    def state(self):
        return [s for conv in (self.conv1, self.conv2) if conv is not None for s in conv.state()] + \
            list(self.mixer.state())

    def forward(self, stream: Stream, step, site) -> Stream:
        k = self.kernels
        h = stream.h
        if h.dtype != torch.float32 or h is stream.origin:       # the stream becomes float32 rows of its own
            h = stream.h = k.widen_rows(h)
        row = None
        if self.passes > 0:
            if site.turn >= self.passes:
                raise ValueError(f"pass {site.turn} of a range that has vectors for {self.passes} passes")
            row = self.step[site.turn]
        terms = _terms(stream.delta)
        waiting = getattr(stream.delta, "row", None)       # a bias the layer before left to add to every row
        if waiting is not None:
            row = waiting if row is None else row + waiting
        stream.delta = stream.stats = None
        if self._fused_filter and step.rows.in_order:      # single tokens: the norms and both filters in one kernel
            second = self.conv2 is not None
            a, b = k.stream_rms_filter(h, terms, row, self.norm1.weight, self.norm2.weight if second else None,
                                       self._one_kernel, self.build.dtype, self.conv1.weight,
                                       self.conv2.weight if second else None, site.slot_state[self.conv1.name],
                                       site.slot_state[self.conv2.name] if second else None, step.slots, step.starts)
            stream.delta = self._pending(a, b, step, site)
            return stream
        if self._one_kernel is not None:
            a, b = k.stream_rms(h, terms, row, self.norm1.weight, self.norm2.weight if self.norm2 is not None else None,
                                self._one_kernel, self.build.dtype)
        else:
            if terms or row is not None:
                k.stream_rms(h, terms, row, None, None, 0.0, self.build.dtype)
            a = self.norm1(h)
            b = self.norm2(h) if self.norm2 is not None else None
        if self.conv1 is not None:
            a = self.conv1(a, step, site)
        if self.ffn is not None and self.conv2 is not None:
            b = self.conv2(b, step, site)
        stream.delta = self._pending(a, b, step, site)
        return stream

    def _pending(self, a, b, step, site) -> Pending:
        """Both sublayers' results from their inputs (one input for both under `shared_norm`), as terms for the next
        norm's kernel. A mixer that names a bias on its last projection (`out_row`, a float32 vector) is asked to
        leave it out (`add_row=False`): it joins the stream in float32, in the same kernel as the terms."""
        row = getattr(self.mixer, "out_row", None)
        out = [self.mixer(a, step, site) if row is None else self.mixer(a, step, site, add_row=False)]
        if self.ffn is not None:
            out.append(self.ffn(a if self.shared_norm else b, step))
        return Pending([(t, 1.0) for t in out], row)

    __call__ = forward
