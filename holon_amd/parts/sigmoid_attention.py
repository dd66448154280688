"""Windowed attention whose weights are sigmoids, not a softmax: a visible key j contributes
sigmoid(q_i . k_j * scale + bias[head]) * v_j to query i, and nothing is normalised over keys. Query i sees keys
i - window + 1 .. i (window 0: all before it). Scores and weights are float32.

Keys and values may differ in width. One page of one site is `[Hkv, P, D]` keys (a token's key is a row) followed by
`[Hkv, V, P]` values (transposed inside the page); with V = D this is the layout of the softmax attention's pages.
HIP forms: `csrc/sigmoid_attention.hip` (any dtype and sizes) and, in bfloat16 with keys and values of one width 64
or 128, the matrix-core prompt and decode kernels of `csrc/attention_mfma.hip` with sigmoid weights in place of
their softmax."""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import FLOAT32, Build, PagedState, Part
from .linear import Linear

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return None if t is None else t.data_ptr()


def head_prepare_plain(qkv, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, table, positions, pages, write_page,
                       write_off, page_size, bias=None, values="own", value_share=1):
    """qkv [T, >= (H + G) D + G' V] (queries, keys, values side by side in the first columns of every row; a row may
    hold more behind them); `bias` (float32, one value a column of q, k and v, or None) is added first. Per head of q
    and k: x * rsqrt(mean(x^2) + eps)
    * weight (when weights are given), then the rotation by `table` [positions, rot] (cos of rot/2 angles, then
    their sines; pairs (i, i + rot/2); dimensions from rot on pass), all in float32 with one rounding. Keys and
    values go into `pages` [pages, G P D + G' P V] (keys [G, P, D], then values [G', V, P]) at (write_page[t],
    write_off[t]); returns q [T, H, D].

    Where the values come from: `values` "own": the G' = G / value_share value heads behind the keys (`value_share`
    key heads read one value head; the page holds G' value heads); "keys": there are no value columns and value head g
    is key head g as projected (bias added; before the norm and the rotation), V = D and G' = G.
    `pages` None: the rows hold queries alone (H D columns) and nothing is stored."""
    t, out_dtype = qkv.shape[0], qkv.dtype
    if pages is None:
        kv_heads = 0
    shared = kv_heads // value_share if values == "own" else 0
    width = (heads + kv_heads) * dim + shared * vdim
    qkv = qkv[:, :width]
    if bias is not None:
        qkv = qkv.float() + bias.float()
    q = qkv[:, : heads * dim].float().view(t, heads, dim)
    k = qkv[:, heads * dim: (heads + kv_heads) * dim].float().view(t, kv_heads, dim)
    if values == "own":
        v = qkv[:, (heads + kv_heads) * dim:].reshape(t, shared, vdim)
    else:
        v = k.clone()
    if q_weight is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_weight.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_weight.float()
    if table is not None:
        rot = table.shape[1]
        cs = table[positions[:t].long()]
        cos, sin = cs[:, None, : rot // 2], cs[:, None, rot // 2:]

        def turn(x):
            a, b = x[..., : rot // 2], x[..., rot // 2: rot]
            return torch.cat((a * cos - b * sin, b * cos + a * sin, x[..., rot:]), dim=-1)
        q, k = turn(q), turn(k)
    if pages is None:
        return q.to(out_dtype)
    keys = pages[:, : kv_heads * page_size * dim].view(-1, kv_heads, page_size, dim)
    vals = pages[:, kv_heads * page_size * dim:].view(-1, v.shape[1], vdim, page_size)
    keys[write_page[:t].long(), :, write_off[:t].long()] = k.to(pages.dtype)
    vals[write_page[:t].long(), :, :, write_off[:t].long()] = v.to(pages.dtype)
    return q.to(pages.dtype)


def _head_prepare_hip(launch, qkv, heads, kv_heads, dim, vdim, q_weight, k_weight, eps, table, positions, pages,
                      write_page, write_off, page_size, bias=None, values="own", value_share=1):
    t, stride = qkv.shape
    if pages is None:
        kv_heads = 0
    from_keys = values == "keys"
    ok = values in ("own", "keys") and value_share >= 1 and kv_heads % value_share == 0 \
        and (not from_keys or (vdim == dim and value_share == 1))
    shared = kv_heads // value_share if ok and not from_keys else 0
    width = (heads + kv_heads) * dim + shared * vdim
    ok = ok and qkv.is_cuda and qkv.is_contiguous() and qkv.dtype in _DT and stride >= width \
        and (pages is None or (pages.dtype == qkv.dtype and pages.is_contiguous() and pages.dim() == 2
                               and pages.shape[1] == kv_heads * page_size * dim
                               + (kv_heads if from_keys else shared) * page_size * vdim
                               and write_page.shape[0] >= t and write_off.shape[0] >= t)) \
        and (q_weight is None) == (k_weight is None) \
        and all(w is None or (w.dtype == qkv.dtype and w.shape == (dim,)) for w in (q_weight, k_weight)) \
        and (table is None or (table.dtype == torch.float32 and table.is_contiguous() and table.shape[1] % 2 == 0
                               and table.shape[1] <= dim)) \
        and positions.shape[0] >= t \
        and (bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.shape == (width,)))
    if not ok:
        raise ValueError(f"head_prepare: qkv {tuple(qkv.shape)} {qkv.dtype}, pages "
                         f"{None if pages is None else tuple(pages.shape)} do not fit {heads}/{kv_heads} heads of "
                         f"{dim}/{vdim}, page {page_size}, values {values!r} shared by {value_share}")
    q = torch.empty((t, heads, dim), dtype=qkv.dtype, device=qkv.device)
    if t:
        launch(qkv.data_ptr(), q.data_ptr(), t, heads, kv_heads, dim, vdim, _ptr(q_weight), _ptr(k_weight), float(eps),
               _ptr(table), table.shape[1] if table is not None else 0, table.shape[0] if table is not None else 0,
               positions.data_ptr(), _ptr(pages), _ptr(write_page) if pages is not None else None,
               _ptr(write_off) if pages is not None else None, page_size,
               pages.shape[0] if pages is not None else 0, _DT[qkv.dtype], _ptr(bias), stride, 1 if from_keys else 0,
               int(value_share))
    return q


def sigmoid_attention_plain(q, pages, table, rows, token_row, positions, kv_heads, vdim, page_size, bias, scale,
                            window, gate):
    """q [T, H, D]; `pages` as `head_prepare` writes them; `table` [S, max_pages] int32; `rows`: the step's rows
    (`AttnRows`); token t belongs to row token_row[t] (slot rows.slots[row]) and stands at positions[t]. bias [H]
    float32 or None. `gate` [T, H V] or None: the result is multiplied by sigmoid(gate). -> [T, H V] in q's dtype;
    the sum over keys runs oldest first."""
    t, heads, dim = q.shape
    keys = pages[:, : kv_heads * page_size * dim].view(-1, kv_heads, page_size, dim)
    vals = pages[:, kv_heads * page_size * dim:].view(-1, kv_heads, vdim, page_size).transpose(2, 3)
    out = torch.zeros((t, heads, vdim), dtype=torch.float32, device=q.device)
    pos = positions.tolist()
    slot_of, rows = rows.slots.tolist(), token_row.tolist()
    group = heads // kv_heads
    for i in range(t):
        first = max(0, pos[i] - window + 1) if window > 0 else 0
        js = torch.arange(first, pos[i] + 1, device=q.device)
        pg = table[slot_of[rows[i]], (js // page_size)].long()
        off = js % page_size
        kk = keys[pg, :, off].float()                                  # [n, G, D]
        vv = vals[pg, :, off].float()                                  # [n, G, V]
        kk = kk.repeat_interleave(group, dim=1)
        vv = vv.repeat_interleave(group, dim=1)
        s = torch.einsum("hd,nhd->nh", q[i].float(), kk) * scale
        if bias is not None:
            s = s + bias.float()
        out[i] = torch.einsum("nh,nhv->hv", torch.sigmoid(s), vv)
    out = out.view(t, heads * vdim)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(q.dtype)


def _sigmoid_attention_hip(launch, q, pages, table, rows, token_row, positions, kv_heads, vdim, page_size, bias,
                           scale, window, gate):
    t, heads, dim = q.shape
    ok = q.is_cuda and q.is_contiguous() and q.dtype in _DT and pages.dtype == q.dtype and pages.is_contiguous() \
        and pages.shape[1] == kv_heads * page_size * (dim + vdim) and table.dtype == torch.int32 \
        and table.is_contiguous() and heads % kv_heads == 0 \
        and (bias is None or (bias.dtype == torch.float32 and bias.shape == (heads,))) \
        and (gate is None or (gate.dtype == q.dtype and gate.is_contiguous() and tuple(gate.shape) == (t, heads * vdim)))
    if not ok:
        raise ValueError(f"sigmoid_attention: q {tuple(q.shape)} {q.dtype}, pages {tuple(pages.shape)} do not fit "
                         f"{kv_heads} kv heads, values of {vdim}, page {page_size}")
    out = torch.empty((t, heads * vdim), dtype=q.dtype, device=q.device)
    general, wide, narrow = launch
    common = (q.data_ptr(), out.data_ptr(), pages.data_ptr(), table.data_ptr(), table.shape[1], rows.slots.data_ptr())
    tail = (heads, kv_heads, dim, vdim, page_size, pages.shape[0], _ptr(bias), float(scale), int(window), _ptr(gate),
            _DT[q.dtype])
    on_cores = q.dtype == torch.bfloat16 and dim == vdim and dim in (64, 128) and page_size % 16 == 0 \
        and heads // kv_heads <= 32 and rows.max_chunk_len <= 4096 * page_size
    if on_cores:      # on the matrix cores: the step's prompt portions in one launch, its decode rows in another
        if rows.n_chunk:
            wide(*common, rows.lens.data_ptr(), rows.query_start.data_ptr(), rows.chunk_rows.data_ptr(), rows.n_chunk,
                 rows.max_chunk_query, rows.max_chunk_len, heads, kv_heads, dim, page_size, float(scale), int(window),
                 _ptr(bias), _ptr(gate))
        if rows.n_decode:
            narrow(*common, rows.lens.data_ptr(), rows.query_start.data_ptr(), rows.decode_rows.data_ptr(),
                   rows.n_decode, rows.max_decode_len, heads, kv_heads, dim, page_size, float(scale), int(window),
                   _ptr(bias), _ptr(gate), int(rows.in_order and rows.n_decode == t))
    else:
        general(*common, token_row.data_ptr(), positions.data_ptr(), None, None, t, *tail)
    return out


register_kernel(KernelOp("head_prepare", head_prepare_plain, "holon_head_prepare",
                         [_P, _P, _I, _I, _I, _I, _I, _P, _P, _F, _P, _I, _I, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I],
                         _head_prepare_hip))
register_kernel(KernelOp("sigmoid_attention", sigmoid_attention_plain,
                         ("holon_sigmoid_attention", "holon_sigmoid_attention_prefill_bf16",
                          "holon_sigmoid_attention_decode_bf16"),
                         ([_P, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _F, _I, _P, _I],
                          [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P],
                          [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P, _I]),
                         _sigmoid_attention_hip))


@register_part("mixer", "sigmoid_window")
class SigmoidWindowAttention(Part):
    """q/k/v projections (one merged product), optional per-head RMS norm on q and k (weights `q_norm`, `k_norm`
    shared by all heads), optional rotary positions, sigmoid-weighted attention inside a window with a bias per head
    (`head_bias`), optional sigmoid output gate read from the mixer's input (`out_gate`), output projection.
    `name` prefixes its state's name among its owner's."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, kv_heads: int, dim: int, vdim: int, hidden: int, layer: int,
                 window: int = 0, scale: float | None = None, qk_norm_eps: float | None = None,
                 position: PartRef | None = None, head_bias: bool = True, out_gate: bool = True,
                 name: str = "") -> None:
        super().__init__(build)
        if heads % kv_heads:
            raise ValueError(f"sigmoid_window: {heads} heads are not a multiple of {kv_heads} kv heads")
        self.heads, self.kv_heads, self.dim, self.vdim, self.hidden = heads, kv_heads, dim, vdim, hidden
        self.window = int(window)
        self.scale = float(scale) if scale is not None else dim ** -0.5
        self.eps = qk_norm_eps
        self.state_name = f"{name}.kv" if name else "kv"
        self.attach("q", Linear(build, inp=hidden, out=heads * dim))
        self.attach("k", Linear(build, inp=hidden, out=kv_heads * dim))
        self.attach("v", Linear(build, inp=hidden, out=kv_heads * vdim))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        if qk_norm_eps is not None:
            self.declare("q_norm", (dim,), init="norm")
            self.declare("k_norm", (dim,), init="norm")
        self.head_bias = head_bias
        if head_bias:
            self.declare("pb", (heads,), kind=FLOAT32, init="zero")
        self.g = None
        if out_gate:
            self.attach("g", Linear(build, inp=hidden, out=heads * vdim))
        self.position = None
        if position is not None:
            self.attach("position", build.make(position, head_dim=dim))
        self.qkv: Linear | None = None

    def state(self):
        return [PagedState(self.state_name, elems=self.kv_heads * (self.dim + self.vdim), window=self.window)]

    def finalize(self) -> None:
        self.qkv = Linear.merge(self.build, self.q, self.k, self.v)
        for name in ("q", "k", "v"):
            self.drop(name)
        self._children["qkv"] = self.qkv

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        held = site.paged[self.state_name]
        view = step.paged[held.group]
        table = getattr(self.position, "table", None)
        q = k.head_prepare(self.qkv(x), self.heads, self.kv_heads, self.dim, self.vdim,
                           getattr(self, "q_norm", None) if self.eps is not None else None,
                           getattr(self, "k_norm", None) if self.eps is not None else None,
                           self.eps or 0.0, table, step.positions, held.pages, view.write_page, view.write_off,
                           view.page_size)
        gate = self.g(x) if self.g is not None else None
        out = k.sigmoid_attention(q, held.pages, view.table, step.rows, step.token_row, step.positions,
                                  self.kv_heads, self.vdim, view.page_size, self.pb if self.head_bias else None,
                                  self.scale, self.window, gate)
        return self.o(out)

    __call__ = forward
