"""Small Dopirax configurations and checkpoints for the tests, and the plain model behind one interface.

The tensors are drawn here, by checkpoint name, from laws that make faults visible: projections keep activations of
order one, the norms' stored weights are spread around zero (the norm multiplies by one plus them), biases, gates and
the vectors behind lam are of order one, the routers' biases reorder the logits, and `sharp` scales the query side so
that few keys carry most of an attention's weight."""
from __future__ import annotations

import copy
import functools
import json
import pathlib

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from tests.plain import dopirax as plain


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def attention(heads, kv_heads, dim, scale, rot=None, base=10000.0, softcap=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def attention_2(heads, kv_heads, dim, vdim, scale, diff, rot=None, base=10000.0, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def model(width, vocab, layers, *, eps=1e-6, scale=2.0):
    return {"architecture": "Dopirax", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "layers": layers}


# A: both mixers and every feed-forward; two layers read the keys and values of layer 1; part of a head turned; keys and
# values of different widths in the differential layers; a layer without feed-forward.
CONFIG_A = model(64, 160, [
    attention(4, 2, 16, 0.3, rot=8, base=100.0, softcap=5.0, mlp=moe(6, 2, 16, shared=24)),
    attention_2(4, 2, 8, 12, 0.35, 0.4, rot=4, base=50.0, mlp=dense(96)),
    attention_2(4, 2, 8, 12, 0.35, 0.4, rot=4, base=50.0, kv_from=1, mlp=moe(5, 1, 16)),
    attention(6, 6, 8, 0.4, rot=8, mlp=None),
    attention_2(4, 2, 8, 12, 0.35, 0.4, rot=4, base=50.0, kv_from=1, mlp=dense(80))])
# B: another order, another eps and scale; a differential layer first with keys and values of one width and every head
# its own kv head; an attention layer with all of a head turned, one without rotation and without a cap; every expert
# chosen; a differential layer without rotation.
CONFIG_B = model(96, 200, [
    attention_2(3, 3, 16, 16, 0.25, 0.7, rot=16, base=500000.0, mlp=moe(4, 4, 16, shared=8)),
    attention(3, 1, 32, 0.2, rot=32, base=1000.0, softcap=15.0, mlp=dense(128)),
    attention_2(6, 2, 8, 24, 0.3, 0.2, mlp=None),
    attention(4, 4, 24, 0.2, mlp=moe(7, 3, 24, shared=40)),
    attention_2(3, 3, 16, 16, 0.25, 0.7, rot=16, base=500000.0, kv_from=0, mlp=dense(64))], eps=1e-5, scale=0.7)
# C: sizes that are 1 or equal: one head, one expert, a scale of 1, two turned dimensions, a diff of 0 (lam is then the
# difference of the two exponentials alone and the gain 1), a head of two values.
CONFIG_C = model(32, 50, [
    attention(1, 1, 8, 1.0, rot=2, mlp=dense(32)),
    attention_2(1, 1, 2, 2, 1.0, 0.0, rot=2, mlp=moe(1, 1, 8, shared=8)),
    attention_2(1, 1, 2, 2, 1.0, 0.0, rot=2, kv_from=1, mlp=None)], scale=1.0)
# D: heads of 64 with keys and values of one width (in bfloat16 on the GPU the matrix-core attention kernels serve
# them), in both mixers; a layer that reads another's keys and values there too.
CONFIG_D = model(96, 120, [
    attention(4, 2, 64, 0.125, rot=32, softcap=20.0, mlp=dense(128)),
    attention_2(2, 1, 64, 64, 0.125, 0.5, rot=64, base=100.0, mlp=moe(8, 2, 32, shared=32)),
    attention_2(2, 1, 64, 64, 0.125, 0.5, rot=64, base=100.0, kv_from=1, mlp=dense(64))])
# One mechanism at a time (the other sublayer absent or as small as it gets).
ONLY_ATTENTION = model(48, 90, [attention(4, 2, 24, 0.2, rot=12, softcap=4.0), attention(3, 1, 8, 0.35, rot=8, base=20.0)])
ONLY_DIFF = model(48, 90, [attention_2(4, 2, 12, 20, 0.3, 0.6, rot=8, base=50.0),
                           attention_2(4, 2, 12, 20, 0.3, 0.6, rot=8, base=50.0, kv_from=0),
                           attention_2(2, 1, 16, 8, 0.25, 0.3, rot=6)])
ONLY_DENSE = model(48, 90, [attention(1, 1, 8, 0.3, mlp=dense(80))])
ONLY_MOE = model(48, 90, [attention(1, 1, 8, 0.3, mlp=moe(12, 4, 16, shared=16))])


def tensor_shapes(c: dict) -> dict[str, tuple[int, ...]]:
    w = c["width"]
    out = {"embed": (c["vocab"], w), "head": (c["vocab"], w), "final.norm": (w,)}
    for i, layer in enumerate(c["layers"]):
        p, m, q = f"l{i}.", layer["mixer"], f"l{i}.mix."
        out[p + "norm1"] = (w,)
        h, g, d, v = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            out.update({q + "q": (h * d, w), q + "q.b": (h * d,), q + "k": (g * d, w), q + "k.b": (g * d,),
                        q + "g": (h, w), q + "o": (w, h * v), q + "o.b": (w,)})
        else:
            out.update({q + "q": (2 * h * d, w), q + "q.norm": (d,), q + "o": (w, h * v)})
            out.update({q + name: (d,) for name in ("lq1", "lk1", "lq2", "lk2")})
            if m.get("kv_from") is None:
                out.update({q + "k": (2 * g * d, w), q + "v": (g * v, w), q + "k.norm": (d,)})
        mlp = layer.get("mlp")
        if not mlp:
            continue
        f = p + "mlp."
        if mlp["kind"] == "dense":
            out.update({f + "up": (mlp["ff"], w), f + "down": (w, mlp["ff"])})
        else:
            ff, experts = mlp["expert"]["ff"], mlp["router"]["experts"]
            for e in range(experts):
                out.update({f"{f}e{e}.gate": (ff, w), f"{f}e{e}.up": (ff, w), f"{f}e{e}.down": (w, ff)})
            out.update({f + "router": (experts, w), f + "router.b": (experts,)})
            if mlp.get("shared"):
                s = mlp["shared"]["ff"]
                out.update({f + "shared.gate": (s, w), f + "shared.up": (s, w), f + "shared.down": (w, s),
                            f + "shared.sg": (1, w)})
    return out


def draw(name: str, shape: tuple[int, ...], g: torch.Generator, sharp: bool) -> torch.Tensor:
    n = lambda: torch.randn(shape, generator=g)               # noqa: E731
    last = name.split(".")[-1]
    if name.endswith("q.norm"):
        x = (4.0 if sharp else 1.0) * (1 + 0.15 * n())
    elif name.endswith("k.norm"):
        x = 1 + 0.15 * n()
    elif last in ("norm1", "norm"):
        x = 0.3 * n()                                         # an offset from one: the norm multiplies by 1 + w
    elif last == "b" and ".mix." in name:
        x = 0.3 * n()
    elif last == "b":                                         # the router's bias
        x = 0.7 * n()
    elif last in ("lq1", "lk1", "lq2", "lk2"):
        x = 0.4 * n()
    elif last in ("router", "sg", "g"):
        x = 3.0 * n() * shape[-1] ** -0.5
    elif last == "embed":
        x = n()
    elif last == "q" and sharp and ".mix." in name and len(shape) == 2:
        x = 4.0 * n() * shape[-1] ** -0.5
    else:
        x = n() * shape[-1] ** -0.5
    return x.bfloat16()


def make_folder(path: pathlib.Path, cfg: dict, seed: int, sharp: bool = False, edit=None) -> pathlib.Path:
    """A model folder for `cfg`. `edit(tensors)` may change the drawn tensors before they are stored."""
    path.mkdir(parents=True, exist_ok=True)
    g = torch.Generator().manual_seed(seed)
    tensors = {name: draw(name, shape, g, sharp) for name, shape in tensor_shapes(cfg).items()}
    if edit is not None:
        edit(tensors)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return path


class PlainDopirax:
    """The plain model of a folder: `logits(ids)` [T, vocab] in float64 arithmetic over the stored weights."""

    def __init__(self, folder: str | pathlib.Path, dtype: torch.dtype = torch.float64, **options) -> None:
        folder = pathlib.Path(folder)
        self.config = json.loads((folder / "config.json").read_text())
        self.dtype, self.options = dtype, options
        self.tensors = {}
        with safe_open(str(folder / "model.safetensors"), "pt") as f:
            for name in f.keys():
                self.tensors[name] = f.get_tensor(name)

    def logits(self, ids: list[int]) -> torch.Tensor:
        return self._logits(tuple(ids))

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids: tuple[int, ...]) -> torch.Tensor:
        return plain.forward(self.config, self.tensors, list(ids), self.dtype, **self.options)[0].float()

    def streams(self, ids: list[int]) -> list[torch.Tensor]:
        return plain.forward(self.config, self.tensors, list(ids), self.dtype, **self.options)[1]


def variant(cfg: dict, **changes) -> dict:
    out = copy.deepcopy(cfg)
    out.update(changes)
    return out
