"""Feed-forward parts. SwiGLU: std/holon_std/ffn/units.py:12-50, activation std/holon_std/ffn/reference.py:7-12.
Beside it a dense feed-forward with the PolyNorm activation and a mixture of experts (HIP forms of their elementwise
steps: `csrc/ffn_kinds.hip`)."""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from .base import FLOAT32, Build, Part, Stream
from .linear import Linear
from .norms import Normed


@register_part("ffn", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)); gate and up are merged into one product after loading (gate rows first)."""

    graph_safe = True

    def __init__(self, build: Build, *, inter: int, hidden: int, layer: int) -> None:
        super().__init__(build)
        self.inter, self.hidden = inter, hidden
        self.attach("gate_proj", Linear(build, inp=hidden, out=inter))
        self.attach("up_proj", Linear(build, inp=hidden, out=inter))
        self.attach("down_proj", Linear(build, inp=inter, out=hidden))
        self.gate_up: Linear | None = None

    def finalize(self) -> None:
        self.gate_up = Linear.merge(self.build, self.gate_proj, self.up_proj)
        self.drop("gate_proj")
        self.drop("up_proj")
        self._children["gate_up"] = self.gate_up

    adds_residual = True

    def absorb_norm(self, norm: Part) -> bool:
        """Fold the norm in front of this part into its first product; it then takes `Normed` input."""
        return self.gate_up.absorb(norm)

    def forward(self, x: torch.Tensor | Normed, step=None, residual: Stream | None = None) -> torch.Tensor | None:
        gate_up, y = self.gate_up, None
        if gate_up.folds(x):
            y = self.kernels.linear_silu_mul(x.h, gate_up.weight, gate_up.tiled, row_scale=gate_up.row_scale(x))
        elif gate_up.reads_folded(x, gated=True):  # 17 to 64 rows: the folded copy over rows normed without the weight
            y = self.kernels.linear_silu_mul(x.unit_value(), gate_up.weight, gate_up.tiled)
        elif gate_up.folded is None:               # fused for steps of few rows
            x = x.value() if isinstance(x, Normed) else x
            y = self.kernels.linear_silu_mul(x, gate_up.weight, gate_up.tiled)
        if y is None:
            y = self.kernels.silu_mul(gate_up(x))
        return self.down_proj(y, residual=residual)

    __call__ = forward


# -- a dense feed-forward with the PolyNorm activation, and a mixture of experts ------------------------------------------
_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise ValueError(what)


def polynorm_plain(z, coef, eps):
    """z [T, F], coef [4] float32 = (a, b, c, e): a N(z) + b N(z^2) + c N(z^3) + e with the powers taken element by
    element and N(v) = v / sqrt(mean(v^2) + eps) over a row. float32 inside, one rounding to z's dtype."""
    x = z.float()
    a, b, c, e = coef.float().unbind(0)

    def unit(v):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (a * unit(x) + b * unit(x * x) + c * unit(x * x * x) + e).to(z.dtype)


def _polynorm_hip(launch, z, coef, eps):
    _need(z.is_cuda and z.is_contiguous() and z.dim() == 2 and z.dtype in _DT and coef.is_cuda and coef.is_contiguous()
          and coef.dtype == torch.float32 and coef.shape == (4,), "polynorm: contiguous rows and four float32 numbers")
    y = torch.empty_like(z)
    if z.shape[0]:
        launch(z.data_ptr(), coef.data_ptr(), y.data_ptr(), z.shape[0], z.shape[1], float(eps), _DT[z.dtype])
    return y


def moe_route_plain(logits, correction, top, groups, keep, scale):
    """Router logits [T, E] float32 -> weights [T, E] float32: s = sigmoid(logits); experts are chosen by s +
    `correction` [E] (None: by s): the `top` largest among the experts of the `keep` best of `groups` equal groups of
    neighbouring experts, a group's score being the sum of its two largest choice scores (groups <= 1: among all).
    A chosen expert's weight is s * scale (the score without the correction, not renormalised), every other 0."""
    s = torch.sigmoid(logits.float())
    choice = s if correction is None else s + correction.float()
    t, e = s.shape
    if groups > 1:
        size = e // groups
        score = choice.view(t, groups, size).topk(min(2, size), dim=-1).values.sum(-1)
        best = score.topk(keep, dim=-1).indices
        open_ = torch.zeros((t, groups), dtype=torch.bool, device=s.device).scatter_(1, best, True)
        choice = choice.masked_fill(~open_.repeat_interleave(size, dim=1), float("-inf"))
    chosen = choice.topk(top, dim=-1).indices
    return torch.zeros_like(s).scatter_(1, chosen, s.gather(1, chosen) * scale)


def _moe_route_hip(launch, logits, correction, top, groups, keep, scale):
    t, e = logits.shape
    _need(logits.is_cuda and logits.is_contiguous() and logits.dtype == torch.float32 and 1 <= top <= e <= 1024
          and (correction is None or (correction.dtype == torch.float32 and correction.is_contiguous()
                                      and correction.shape == (e,)))
          and (groups <= 1 or (e % groups == 0 and 1 <= keep <= groups)),
          f"moe_route: {e} experts, top {top}, {groups} groups of which {keep} (float32 logits, at most 1,024 experts)")
    w = torch.empty_like(logits)
    if t:
        launch(logits.data_ptr(), None if correction is None else correction.data_ptr(), w.data_ptr(), t, e, int(top),
               int(groups), int(keep), float(scale))
    return w


def moe_router_plain(x, router, correction, top, groups, keep, scale):
    """x [T, W] (any dtype), router [E, W] float32: the float32 logits x . router[e], then `moe_route` on them."""
    return moe_route_plain(x.float() @ router.float().T, correction, top, groups, keep, scale)


def _moe_router_hip(launch, x, router, correction, top, groups, keep, scale):
    (t, w), e = x.shape, router.shape[0]
    _need(x.is_cuda and x.is_contiguous() and x.dtype in _DT and router.is_contiguous() and router.dtype == torch.float32
          and router.shape == (e, w) and 1 <= top <= e <= 1024 and w <= 12288
          and (correction is None or (correction.dtype == torch.float32 and correction.is_contiguous()
                                      and correction.shape == (e,)))
          and (groups <= 1 or (e % groups == 0 and 1 <= keep <= groups)),
          f"moe_router: rows {tuple(x.shape)} {x.dtype}, {e} experts, top {top}, {groups} groups of which {keep}")
    weights = torch.empty((t, e), dtype=torch.float32, device=x.device)
    if t:
        launch(x.data_ptr(), router.data_ptr(), None if correction is None else correction.data_ptr(),
               weights.data_ptr(), t, w, e, int(top), int(groups), int(keep), float(scale), _DT[x.dtype])
    return weights


def moe_gate_plain(gate_up, weights, ff, shared, shared_weight=False):
    """gate_up [T, 2 C] with C = E ff + shared columns of gates, then as many of ups; weights [T, E] float32.
    -> [T, C]: silu(gate) * up (as `silu_mul` rounds it), times the weight of the column's expert (column c belongs to
    expert c // ff; the last `shared` columns to an expert that every token uses with weight 1); exactly 0 where the
    weight is 0. One more rounding for the weight. `shared_weight`: weights is [T, E + 1] and its last column is the
    weight of the shared expert's columns."""
    t, e = weights.shape[0], weights.shape[1] - int(bool(shared_weight))
    c = e * ff + shared
    g, u = gate_up[:, :c].float(), gate_up[:, c:].float()
    act = ((g * torch.sigmoid(g)).to(gate_up.dtype).float() * u).to(gate_up.dtype)
    w = weights[:, :e].repeat_interleave(ff, dim=1)
    if shared:
        last = weights[:, e:].expand(t, shared) if shared_weight else torch.ones((t, shared), dtype=w.dtype, device=w.device)
        w = torch.cat((w, last), dim=1)
    return torch.where(w == 0, torch.zeros_like(act), (act.float() * w).to(gate_up.dtype))


def _moe_gate_hip(launch, gate_up, weights, ff, shared, shared_weight=False):
    t, e = weights.shape[0], weights.shape[1] - int(bool(shared_weight))
    c = e * ff + shared
    _need(gate_up.is_cuda and gate_up.is_contiguous() and gate_up.dtype in _DT and gate_up.shape == (t, 2 * c)
          and weights.is_contiguous() and weights.dtype == torch.float32 and e >= 1,
          f"moe_gate: rows {tuple(gate_up.shape)} for {e} experts of {ff} and {shared} shared columns")
    y = torch.empty((t, c), dtype=gate_up.dtype, device=gate_up.device)
    if t:
        launch(gate_up.data_ptr(), weights.data_ptr(), y.data_ptr(), t, e, ff, shared, _DT[gate_up.dtype],
               weights.shape[1], e if shared_weight else -1)
    return y


def moe_router_top_plain(x, router, bias, experts, top):
    """x [T, W] (any dtype), router [R, W] float32 with R = experts or experts + 1, bias [experts] float32 or None:
    the float32 logits z = x . router[e] + bias[e]; the `top` largest are chosen (equal ones: the lower index first)
    and weighted by the softmax over the chosen logits alone, every other expert 0. A last row beyond the experts is a
    gate: its column holds sigmoid(x . router[experts]). -> [T, R] float32."""
    z = x.float() @ router.float().T
    logits = z[:, :experts] + (bias.float() if bias is not None else 0.0)
    order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :top]
    chosen = logits.gather(1, order)
    w = torch.zeros_like(logits).scatter_(1, order, torch.softmax(chosen, dim=-1))
    return torch.cat((w, torch.sigmoid(z[:, experts:])), dim=1).contiguous()


def _moe_router_top_hip(launch, x, router, bias, experts, top):
    (t, w), r = x.shape, router.shape[0]
    _need(x.is_cuda and x.is_contiguous() and x.dtype in _DT and router.is_contiguous() and router.dtype == torch.float32
          and router.shape == (r, w) and r in (experts, experts + 1) and 1 <= top <= experts <= 1024 and w <= 12288
          and (bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.shape == (experts,))),
          f"moe_router_top: rows {tuple(x.shape)} {x.dtype}, router {tuple(router.shape)}, top {top} of {experts}")
    weights = torch.empty((t, r), dtype=torch.float32, device=x.device)
    if t:
        launch(x.data_ptr(), router.data_ptr(), None if bias is None else bias.data_ptr(), weights.data_ptr(), t, w,
               experts, r, int(top), _DT[x.dtype])
    return weights


def relu2_plain(z):
    """z [T, F] -> max(z, 0)^2, float32 inside, one rounding."""
    return torch.relu(z.float()).pow(2).to(z.dtype)


def _relu2_hip(launch, z):
    _need(z.is_cuda and z.is_contiguous() and z.dtype in _DT, "relu2: contiguous float32 or bfloat16 values on the GPU")
    y = torch.empty_like(z)
    if z.numel():
        launch(z.data_ptr(), y.data_ptr(), z.numel(), _DT[z.dtype])
    return y


register_kernel(KernelOp("polynorm", polynorm_plain, "holon_polynorm", [_P, _P, _P, _L, _I, _F, _I], _polynorm_hip))
register_kernel(KernelOp("moe_route", moe_route_plain, "holon_moe_route", [_P, _P, _P, _L, _I, _I, _I, _I, _F],
                         _moe_route_hip))
register_kernel(KernelOp("moe_router", moe_router_plain, "holon_moe_router",
                         [_P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _F, _I], _moe_router_hip))
register_kernel(KernelOp("moe_gate", moe_gate_plain, "holon_moe_gate", [_P, _P, _P, _L, _I, _I, _I, _I, _I, _I],
                         _moe_gate_hip))
register_kernel(KernelOp("moe_router_top", moe_router_top_plain, "holon_moe_router_top",
                         [_P, _P, _P, _P, _L, _I, _I, _I, _I, _I], _moe_router_top_hip))
register_kernel(KernelOp("relu2", relu2_plain, "holon_relu2", [_P, _P, _L, _I], _relu2_hip))


def linear_relu2_plain(x, weight, tiled=None):
    """relu2(x W^T) where one kernel does both, with the roundings of the two one after the other; None where it does
    not (the caller then composes them). The plain form never does."""
    return None


def _linear_relu2_hip(launch, x, weight, tiled=None):
    """Steps of up to 16 bfloat16 rows: the few-row product with the activation in its epilogue."""
    (m, k), n = x.shape, weight.shape[0]
    if not (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.is_contiguous()
            and weight.is_contiguous() and weight.shape[1] == k and 1 <= m <= 16 and n % 16 == 0 and k % 32 == 0
            and k >= 256 and (tiled is None or (tiled.shape == weight.shape and tiled.dtype == weight.dtype
                                                 and tiled.is_contiguous()))):
        return None
    y = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    launch(x.data_ptr(), (tiled if tiled is not None else weight).data_ptr(), y.data_ptr(), m, n, k, 4,
           int(tiled is not None))
    return y


register_kernel(KernelOp("linear_relu2", linear_relu2_plain, "holon_gemm_skinny_bf16", [_P, _P, _P, _I, _I, _I, _I, _I],
                         _linear_relu2_hip))


@register_part("ffn", "polynorm")
class PolyNormFFN(Part):
    """down(act(up(x))) with act = a N(z) + b N(z^2) + c N(z^3) + e (`act` holds a, b, c, e; N divides a token's
    vector by its root mean square, `eps` inside the root)."""

    graph_safe = True

    def __init__(self, build: Build, *, inter: int, eps: float, hidden: int, layer: int) -> None:
        super().__init__(build)
        self.inter, self.hidden, self.eps = inter, hidden, float(eps)
        self.attach("up_proj", Linear(build, inp=hidden, out=inter))
        self.attach("down_proj", Linear(build, inp=inter, out=hidden))
        self.declare("act", (4,), kind=FLOAT32, init="unit")

    def forward(self, x: torch.Tensor, step=None) -> torch.Tensor:
        return self.down_proj(self.kernels.polynorm(self.up_proj(x), self.act, self.eps))

    __call__ = forward


@register_part("ffn", "dense")
class DenseFFN(Part):
    """down(act(up(x))) with an activation by name: `relu2`, the square of max(z, 0)."""

    graph_safe = True
    ACTS = ("relu2",)

    def __init__(self, build: Build, *, inter: int, hidden: int, layer: int, act: str = "relu2") -> None:
        super().__init__(build)
        if act not in self.ACTS:
            raise ValueError(f"ffn dense: no activation {act!r} ({', '.join(self.ACTS)})")
        self.inter, self.hidden, self.act = inter, hidden, act
        self.attach("up_proj", Linear(build, inp=hidden, out=inter))
        self.attach("down_proj", Linear(build, inp=inter, out=hidden))

    def forward(self, x: torch.Tensor, step=None) -> torch.Tensor:
        up = self.up_proj
        y = self.kernels.linear_relu2(x, up.weight, up.tiled if up.folded is None else None)
        if y is None:
            y = self.kernels.relu2(up(x))
        return self.down_proj(y)

    __call__ = forward


@register_part("ffn", "moe")
class MoE(Part):
    """A mixture of SiLU-gated experts with a router, and an optional shared expert that every token uses.

    `score` "softmax_top" is the other router: float32 logits z = W_r x + b (`router_bias`), the `top` largest z are
    chosen and weighted by the softmax over the chosen z alone (no groups, no scale). `shared_gated`: the shared
    expert's output is multiplied by sigmoid(w_sg . x), one number a token; w_sg rides as one more row of the router's
    weights, so the router's kernel leaves that weight too. What follows describes `score` "sigmoid".

    Router: float32 logits (products of the input as it is with float32 weights, summed in float32), scores s =
    sigmoid(logits); experts are chosen by s + `correction` (`bias`), optionally
    only within the `keep` best of `groups` groups of neighbouring experts, `top` per token; a chosen expert's output
    is weighted by s * `scale`. All experts' gate and up projections are one product and all down projections
    another: the activations of experts a token did not choose are set to 0 in between (`moe_gate`), so the second
    product adds up exactly the chosen experts' weighted outputs, and the shared expert's columns ride in the same two
    products. Every step launches the same kernels whatever was chosen."""

    graph_safe = True

    def __init__(self, build: Build, *, experts: int, top: int, inter: int, hidden: int, layer: int,
                 scale: float = 1.0, groups: int = 1, keep: int = 1, bias: bool = True, shared: int = 0,
                 score: str = "sigmoid", shared_gated: bool = False) -> None:
        super().__init__(build)
        if not 1 <= top <= experts:
            raise ValueError(f"moe: top {top} of {experts} experts")
        if score not in ("sigmoid", "softmax_top"):
            raise ValueError(f"moe: no router score {score!r} (sigmoid, softmax_top)")
        if score == "softmax_top" and (groups > 1 or float(scale) != 1.0):
            raise ValueError("moe: the softmax over the chosen logits comes without groups and without a scale")
        if shared_gated and (not shared or score != "softmax_top"):
            raise ValueError("moe: a gate on the shared expert needs a shared expert and the softmax_top router")
        self.score, self.shared_gated = score, bool(shared_gated)
        if groups > 1 and (experts % groups or not 1 <= keep <= groups or top > keep * (experts // groups)):
            raise ValueError(f"moe: {experts} experts in {groups} groups, {keep} kept, top {top}")
        self.experts, self.top, self.inter, self.hidden, self.shared = experts, top, inter, hidden, int(shared)
        self.scale, self.groups, self.keep = float(scale), int(groups), int(keep)
        self.declare("router", (experts, hidden), kind=FLOAT32)
        self.has_bias = bool(bias)
        if self.has_bias:
            # (sigmoid: a correction of the choice alone; softmax_top: the logits' bias)
            self.declare("correction" if score == "sigmoid" else "router_bias", (experts,), kind=FLOAT32, init="zero")
        if self.shared_gated:
            self.declare("shared_sg", (1, hidden), kind=FLOAT32)
        self.declare("gate", (experts, inter, hidden))
        self.declare("up", (experts, inter, hidden))
        self.declare("down", (experts, hidden, inter))
        if self.shared:
            self.declare("shared_gate", (self.shared, hidden))
            self.declare("shared_up", (self.shared, hidden))
            self.declare("shared_down", (hidden, self.shared))
        self.gate_up: Linear | None = None
        self.all_down: Linear | None = None

    def finalize(self) -> None:
        if self.gate is None:
            return
        if self.shared_gated and self.router.shape[0] == self.experts:
            self.router = torch.cat((self.router, self.shared_sg)).contiguous()
            del self._decls["shared_sg"]
            self.shared_sg = None
        e, f, w = self.experts, self.inter, self.hidden
        cols = e * f + self.shared
        gate_up, down = Linear(self.build, inp=w, out=2 * cols), Linear(self.build, inp=cols, out=w)
        gates, ups = [self.gate.reshape(e * f, w)], [self.up.reshape(e * f, w)]
        downs = [self.down.permute(1, 0, 2).reshape(w, e * f)]
        if self.shared:
            gates.append(self.shared_gate)
            ups.append(self.shared_up)
            downs.append(self.shared_down)
        gate_up.weight = torch.cat(gates + ups, dim=0).contiguous()
        down.weight = torch.cat(downs, dim=1).contiguous()
        for name in ("gate", "up", "down", "shared_gate", "shared_up", "shared_down"):
            if name in self._decls:
                del self._decls[name]
                setattr(self, name, None)
        gate_up.finalize()
        down.finalize()
        self.gate_up = self.attach("gate_up", gate_up)
        self.all_down = self.attach("all_down", down)

    def forward(self, x: torch.Tensor, step=None) -> torch.Tensor:
        k = self.kernels
        if self.score == "softmax_top":
            weights = k.moe_router_top(x, self.router, self.router_bias if self.has_bias else None, self.experts,
                                       self.top)
            act = k.moe_gate(self.gate_up(x), weights, self.inter, self.shared, shared_weight=self.shared_gated)
            return self.all_down(act)
        weights = k.moe_router(x, self.router, self.correction if self.has_bias else None, self.top, self.groups,
                               self.keep, self.scale)
        act = k.moe_gate(self.gate_up(x), weights, self.inter, self.shared)
        return self.all_down(act)

    __call__ = forward
