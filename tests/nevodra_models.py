"""Small Nevodra configurations and checkpoints for the tests, and the plain model behind one interface.

The tensors are drawn here, by checkpoint name, from laws that make faults visible: projections keep activations of
order one, norm weights and filter taps are far from the identity, sinks and distance biases are of the order of the
scores, the router's corrections push some choice scores below zero, and `sharp` scales the query side so that few
keys carry most of the attention's weight."""
from __future__ import annotations

import copy
import functools
import json
import pathlib

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from tests.plain import nevodra as plain


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale, groups=None, shared=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def attention(heads, kv_heads, dim, vdim, scale, size=None, keep_first=0, softcap=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        m["mask"] = {"size": size, "keep_first": keep_first}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, rot_dims=None, base=10000.0, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}
    if rot_dim:
        m["rot"] = {"dims": rot_dims or rot_dim, "base": base}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def model(width, vocab, layers, *, eps=1e-6, scale=2.0, taps=3, loop=None):
    out = {"architecture": "Nevodra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "embedding": {"scale": scale},
           "layers": layers}
    if taps:
        out["canon"] = {"taps": taps}
    if loop:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# A: both mixers and both feed-forwards; the two middle layers run three times; a window of 9 with 3 kept tokens (below
# every page size used); keys and values of different widths; part of the rotated dimensions rotated; two of four
# groups kept.
CONFIG_A = model(64, 160, [
    latent(4, 16, 8, 12, 24, 0.2, rot_dims=4, base=100.0, mlp=dense(96)),
    attention(4, 2, 16, 24, 0.25, size=9, keep_first=3, softcap=6.0, mlp=moe(8, 3, 16, 1.5, groups=(4, 2), shared=24)),
    latent(2, 8, 16, 16, 40, 0.3, mlp=moe(6, 2, 24, 2.5)),
    attention(6, 6, 8, 8, 0.35, size=33, keep_first=17, mlp=dense(80))], taps=3, loop=(1, 3, 3))
# B: another order, no loop, four taps, a layer without feed-forward; windows of 16 (a page) and 40 with as many kept
# tokens as a page holds; a router without groups and without a shared expert; one expert a token.
CONFIG_B = model(96, 200, [
    attention(3, 1, 32, 16, 0.2, size=16, keep_first=1, mlp=moe(5, 1, 32, 1.0)),
    latent(3, 16, 16, 8, 32, 0.25, base=500000.0, mlp=None),
    attention(4, 4, 24, 24, 0.2, size=40, keep_first=16, softcap=15.0, mlp=dense(128)),
    latent(6, 8, 4, 16, 16, 0.3, rot_dims=2, mlp=moe(4, 4, 16, 0.5, groups=(2, 2), shared=8))], eps=1e-5, scale=0.7,
    taps=4)
# C: sizes that are 1 or equal: one head, a window of one token, one tap (the filter sees the token itself), a scale of
# 1, a loop that runs once and covers the whole model, no kept tokens, full attention without a mask, one group.
CONFIG_C = model(32, 50, [
    attention(1, 1, 8, 8, 1.0, size=1, mlp=dense(32)),
    latent(1, 8, 2, 8, 8, 1.0, mlp=moe(2, 1, 8, 1.0, groups=(1, 1))),
    attention(2, 1, 8, 8, 0.5, mlp=None)], scale=1.0, taps=1, loop=(0, 3, 1))
# D: the loop opens at the first layer (its vector joins the embedding's rows) and closes before the last; two taps;
# heads of 64 with keys and values of one width; a latent whose cache entry is 128 wide.
CONFIG_D = model(96, 120, [
    attention(4, 2, 64, 64, 0.125, size=50, keep_first=4, softcap=20.0, mlp=dense(128)),
    latent(4, 32, 32, 32, 96, 0.15, mlp=moe(8, 2, 32, 2.0, groups=(2, 1), shared=32)),
    latent(2, 16, 0, 16, 32, 0.25, mlp=dense(64))], taps=2, loop=(0, 2, 2))
# One mechanism at a time (the other sublayer absent or as small as it gets).
ONLY_ATTENTION = model(48, 90, [attention(4, 2, 24, 12, 0.2, size=12, keep_first=2, softcap=4.0),
                                attention(3, 1, 8, 16, 0.35)], taps=0)
ONLY_LATENT = model(48, 90, [latent(4, 12, 8, 20, 24, 0.2, base=50.0), latent(2, 16, 6, 8, 8, 0.25, rot_dims=4)], taps=0)
ONLY_DENSE = model(48, 90, [latent(1, 8, 2, 8, 8, 0.3, mlp=dense(80))], taps=0)
ONLY_MOE = model(48, 90, [latent(1, 8, 2, 8, 8, 0.3, mlp=moe(12, 4, 16, 2.0, groups=(3, 2), shared=16))], taps=0)
ONLY_FILTER = model(48, 90, [latent(1, 8, 2, 8, 8, 0.3, mlp=dense(48))], taps=5, loop=(0, 1, 2))


def tensor_shapes(c: dict) -> dict[str, tuple[int, ...]]:
    w, taps = c["width"], (c.get("canon") or {}).get("taps", 0)
    out = {"embed": (c["vocab"], w), "head": (c["vocab"], w), "final.norm": (w,)}
    if c.get("loop"):
        out["loop.step"] = (c["loop"]["times"], w)
    for i, layer in enumerate(c["layers"]):
        p, m, q = f"l{i}.", layer["mixer"], f"l{i}.mix."
        out[p + "norm1"] = (w,)
        if taps:
            out[p + "canon1"] = (w, taps)
        if layer["type"] == "attention":
            h, g, d, v = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({q + "q": (h * d, w), q + "k": (g * d, w), q + "v": (g * v, w), q + "q.norm": (h * d,),
                        q + "k.norm": (g * d,), q + "r1": (h,), q + "r2": (h,), q + "o": (w, h * v)})
        else:
            h, d, r, v, kr = m["heads"], m["dim"], m.get("rot_dim", 0), m["vdim"], m["kv_rank"]
            out.update({q + "q": (h * (d + r), w), q + "dkv": (kr + r, w), q + "dkv.norm": (kr,), q + "uk": (h * d, kr),
                        q + "uv": (h * v, kr), q + "sink": (h,), q + "o": (w, h * v)})
        mlp = layer.get("mlp")
        if not mlp:
            continue
        out[p + "norm2"] = (w,)
        if taps:
            out[p + "canon2"] = (w, taps)
        f = p + "mlp."
        if mlp["kind"] == "dense":
            out.update({f + "up": (mlp["ff"], w), f + "down": (w, mlp["ff"]), f + "act": (4,)})
        else:
            ff, experts = mlp["expert"]["ff"], mlp["router"]["experts"]
            for e in range(experts):
                out.update({f"{f}e{e}.gate": (ff, w), f"{f}e{e}.up": (ff, w), f"{f}e{e}.down": (w, ff)})
            out.update({f + "router": (experts, w), f + "correction": (experts,)})
            if mlp.get("shared"):
                s = mlp["shared"]["ff"]
                out.update({f + "shared.gate": (s, w), f + "shared.up": (s, w), f + "shared.down": (w, s)})
    return out


def draw(name: str, shape: tuple[int, ...], g: torch.Generator, sharp: bool) -> torch.Tensor:
    n = lambda: torch.randn(shape, generator=g)               # noqa: E731
    u = lambda: torch.rand(shape, generator=g)                # noqa: E731
    last = name.split(".")[-1]
    if last == "norm" and name.endswith("q.norm") and sharp:
        x = 4.0 * (1 + 0.15 * n())
    elif last in ("norm", "norm1", "norm2"):
        x = 1 + 0.15 * n()
    elif last in ("canon1", "canon2"):
        x = 0.3 * n()
    elif last == "step":
        x = 0.5 * n()
    elif last == "r1":
        x = u()
    elif last == "r2":
        x = 2.0 * u()
    elif last == "sink":
        x = 1.5 * n()
    elif last == "act":
        x = torch.tensor([0.9, 0.4, -0.3, 0.1]) + 0.2 * n()
    elif last == "correction":
        x = 0.5 * n() - 0.4                                   # some choice scores fall below zero
    elif last == "router":
        x = 3.0 * n() * shape[-1] ** -0.5
    elif last == "embed":
        x = n()
    elif last == "q" and sharp and ".mix." in name:
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


class PlainNevodra:
    """The plain model of a folder: `logits(ids)` [T, vocab] in float64 arithmetic over the stored weights."""

    def __init__(self, folder: str | pathlib.Path, dtype: torch.dtype = torch.float64) -> None:
        folder = pathlib.Path(folder)
        self.config = json.loads((folder / "config.json").read_text())
        self.dtype = dtype
        self.tensors = {}
        with safe_open(str(folder / "model.safetensors"), "pt") as f:
            for name in f.keys():
                self.tensors[name] = f.get_tensor(name)

    def logits(self, ids: list[int]) -> torch.Tensor:
        return self._logits(tuple(ids))

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids: tuple[int, ...]) -> torch.Tensor:
        return plain.forward(self.config, self.tensors, list(ids), self.dtype)[0].float()

    def streams(self, ids: list[int]) -> list[torch.Tensor]:
        return plain.forward(self.config, self.tensors, list(ids), self.dtype)[1]


def variant(cfg: dict, **changes) -> dict:
    out = copy.deepcopy(cfg)
    out.update(changes)
    return out
