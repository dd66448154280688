"""A residual stream that is kept in float32 whatever the engine's dtype: the layer norm that reads it, the pre-norm
block that owns it, and the few elementwise operations around it (their HIP forms are in `csrc/stream32.hip`).

The block is for designs that ask for a 32-bit residual sum: every term a mixer or a feed-forward produces is added
into float32 rows, each add is fused into the norm that reads the sum, and what the norm hands on is in the engine's
dtype again. Beside that the block knows three optional things, each a parameter: a short causal filter on the normed
input of the mixer (`conv_taps`), a layer without feed-forward (`ffn=None`), and a projection of [stream; embedding
rows] in front of the layer (`reentry`), for models that run a range of layers several times and feed the embedding
in again at the start of each pass.
"""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import Build, NormPart, Part, Stream
from .convs import CausalConv
from .linear import Linear

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return None if t is None else t.data_ptr()


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise ValueError(what)


# -- operations -------------------------------------------------------------------------------------------------------
def widen_rows_plain(x):
    """x [T, W] -> a new float32 tensor of the same values."""
    return x.to(torch.float32, copy=True)


def _widen_rows_hip(launch, x):
    _need(x.is_cuda and x.is_contiguous() and x.dtype in _DT, "widen_rows: contiguous float32 or bfloat16 rows on the GPU")
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    launch(x.data_ptr(), y.data_ptr(), x.numel(), _DT[x.dtype])
    return y


def stream_norm_plain(x32, terms, weight, eps, out_dtype):
    """x32 [T, W] float32 += sum of scale * term over `terms` [(tensor [T, W], scale)], in place, float32 arithmetic in
    the order given. Then, with `weight` [W]: returns (x - mean) / sqrt(var + eps) * weight of the rows, in
    `out_dtype` (biased variance, two passes, float32 inside); without: returns None."""
    for term, scale in terms:
        x32.add_(term.float() * scale)
    if weight is None:
        return None
    mu = x32.mean(-1, keepdim=True)
    d = x32 - mu
    return (d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(out_dtype)


def _stream_norm_hip(launch, x32, terms, weight, eps, out_dtype):
    _need(x32.is_cuda and x32.is_contiguous() and x32.dtype == torch.float32 and x32.dim() == 2,
          "stream_norm: the stream is contiguous float32 rows on the GPU")
    _need(len(terms) <= 2, "stream_norm: at most two terms")
    rows, dim = x32.shape
    ptrs, scales, dts = [None, None], [0.0, 0.0], [0, 0]
    for i, (term, scale) in enumerate(terms):
        _need(term.is_cuda and term.is_contiguous() and term.shape == x32.shape and term.dtype in _DT,
              f"stream_norm: term {i} must be contiguous rows of the stream's shape")
        ptrs[i], scales[i], dts[i] = term.data_ptr(), float(scale), _DT[term.dtype]
    y = None
    if weight is not None:
        _need(weight.is_cuda and weight.is_contiguous() and weight.shape == (dim,) and weight.dtype == out_dtype
              and out_dtype in _DT, "stream_norm: a weight of the rows' width, in the output's dtype")
        y = torch.empty((rows, dim), dtype=out_dtype, device=x32.device)
    launch(x32.data_ptr(), ptrs[0], scales[0], dts[0], ptrs[1], scales[1], dts[1], _ptr(weight), _ptr(y), rows, dim,
           float(eps), _DT[out_dtype] if weight is not None else 0)
    return y


def pair_rows_plain(x32, origin, out_dtype):
    """[x32 | origin] side by side -> [T, W1 + W2] in `out_dtype`."""
    return torch.cat((x32.to(out_dtype), origin.to(out_dtype)), dim=-1)


def _pair_rows_hip(launch, x32, origin, out_dtype):
    _need(x32.is_cuda and x32.is_contiguous() and x32.dtype == torch.float32 and origin.is_contiguous()
          and origin.dtype in _DT and origin.shape[0] == x32.shape[0] and out_dtype in _DT,
          "pair_rows: float32 rows and as many rows of the embedding")
    y = torch.empty((x32.shape[0], x32.shape[1] + origin.shape[1]), dtype=out_dtype, device=x32.device)
    launch(x32.data_ptr(), origin.data_ptr(), y.data_ptr(), x32.shape[0], x32.shape[1], origin.shape[1],
           _DT[origin.dtype], _DT[out_dtype])
    return y


def softcap_plain(logits, cap):
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    logits.copy_(cap * torch.tanh(logits / cap))
    return logits


def _softcap_hip(launch, logits, cap):
    _need(logits.is_cuda and logits.is_contiguous() and logits.dtype == torch.float32, "softcap: float32 logits on the GPU")
    launch(logits.data_ptr(), logits.numel(), float(cap))
    return logits


register_kernel(KernelOp("widen_rows", widen_rows_plain, "holon_widen_rows", [_P, _P, _L, _I], _widen_rows_hip))
register_kernel(KernelOp("stream_norm", stream_norm_plain, "holon_stream_norm",
                         [_P, _P, _F, _I, _P, _F, _I, _P, _P, _L, _I, _F, _I], _stream_norm_hip))
register_kernel(KernelOp("pair_rows", pair_rows_plain, "holon_pair_rows", [_P, _P, _P, _L, _I, _I, _I, _I],
                         _pair_rows_hip))
register_kernel(KernelOp("softcap", softcap_plain, "holon_softcap", [_P, _L, _F], _softcap_hip))


# -- parts ------------------------------------------------------------------------------------------------------------
class Pending:
    """Terms not yet added to a float32 stream: [(tensor [T, W], scale)], and optionally `row`, one float32 vector [W]
    that is added to every row (a projection's bias that waits for the same add). The next norm's kernel adds them as
    it reads the rows; a norm whose kernel takes no such vector is not handed one."""

    def __init__(self, terms: list[tuple[torch.Tensor, float]], row: torch.Tensor | None = None) -> None:
        self.terms, self.row = terms, row

    def index_select(self, dim: int, index: torch.Tensor) -> "Pending":
        if dim != 0:
            raise ValueError("Pending.index_select: rows only (dim 0)")
        return Pending([(t.index_select(0, index), s) for t, s in self.terms], self.row)


def _terms(x) -> list[tuple[torch.Tensor, float]]:
    if x is None:
        return []
    return x.terms if isinstance(x, Pending) else [(x, 1.0)]


@register_part("norm", "layernorm")
class LayerNorm(NormPart):
    """y = (x - mean) / sqrt(var + eps) * weight over the last `dim` values, no bias; float32 inside, the result in
    the engine's dtype. It reads float32 rows (a 32-bit residual stream) or rows in the engine's dtype."""

    graph_safe = True

    def __init__(self, build: Build, *, eps: float, dim: int) -> None:
        super().__init__(build)
        self.eps, self.dim = float(eps), dim
        self.declare("weight", (dim,), init="norm")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dtype != torch.float32:
            x = self.kernels.widen_rows(x)
        return self.kernels.stream_norm(x, [], self.weight, self.eps, self.build.dtype)

    __call__ = forward

    def add(self, x, residual: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """(norm(residual + x), residual + x): `residual` is float32 and takes the sum in place; `x` is a tensor or
        `Pending` terms with their scales."""
        return self.kernels.stream_norm(residual, _terms(x), self.weight, self.eps, self.build.dtype), residual


@register_part("block", "prenorm32")
class PreNorm32(Part):
    """h += mixer(filter(norm1(h))); h += ffn(norm2(h)), with h in float32. `filter` (conv_taps > 0) replaces the
    normed rows a by a + conv(a), a causal filter over time on each channel whose last taps - 1 inputs are part of
    the request's state. A mixer may answer with `Pending` terms (several results with their scales); every add
    happens inside the kernel of the norm that reads the sum, the layer's last one in the next reader's norm."""

    graph_safe = True
    reads_origin = False

    def __init__(self, build: Build, *, layer: int, hidden: int, mixer: PartRef, ffn: PartRef | None, norm: PartRef,
                 conv_taps: int = 0, reentry: bool = False) -> None:
        super().__init__(build)
        self.hidden = hidden
        self.attach("norm1", build.make(norm, dim=hidden))
        self.attach("mixer", build.make(mixer, layer=layer, hidden=hidden))
        self.conv = None
        if conv_taps > 0:
            self.attach("conv", CausalConv(build, channels=hidden, taps=conv_taps, add_input=True, name="filter"))
        self.ffn = None
        if ffn is not None:
            self.attach("norm2", build.make(norm, dim=hidden))
            self.attach("ffn", build.make(ffn, layer=layer, hidden=hidden))
        self.entry = None
        if reentry:
            self.reads_origin = True
            self.attach("entry", Linear(build, inp=2 * hidden, out=hidden))

    def state(self):
        return (self.conv.state() if self.conv is not None else []) + list(self.mixer.state())

    def forward(self, stream: Stream, step, site) -> Stream:
        k = self.kernels
        h = stream.h
        if h.dtype != torch.float32 or h is stream.origin:       # the first block: the stream becomes float32 rows of
            h = stream.h = k.widen_rows(h)                       # its own (the embedding's rows stay as they are)
        if self.entry is not None:
            k.stream_norm(h, _terms(stream.delta), None, 0.0, self.build.dtype)
            stream.delta = None
            both = k.pair_rows(h, stream.origin, self.build.dtype)
            h = stream.h = self.entry(both, out_dtype=torch.float32)
        a = self.norm1.add(stream.delta, h)[0]
        stream.delta = stream.stats = None
        if self.conv is not None:
            a = self.conv(a, step, site)
        mixed = self.mixer(a, step, site)
        if self.ffn is None:
            stream.delta = mixed if isinstance(mixed, Pending) else Pending(_terms(mixed))
            return stream
        x = self.norm2.add(mixed, h)[0]
        stream.delta = Pending(_terms(self.ffn(x, step)))
        return stream

    __call__ = forward
