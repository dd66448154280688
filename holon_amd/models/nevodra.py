"""Nevodra: its typed configuration, and configuration to spec.

A decoder whose layers add both sublayers' results to the same residual stream, x += mixer(f(norm1(x))) +
ffn(f(norm2(x))), the stream kept in float32, with RMS norms and a short causal filter f (a + conv(a)) on what each
sublayer reads. The embedding's rows are multiplied by a constant. Each layer names its mixer: `attention`
(grouped-query softmax attention without rotation: one RMS norm over all query values and one over all key values,
scores squashed by a tanh cap, a logarithmic distance bias per head, a sliding window that keeps the first tokens
visible) or `latent_attention` (keys and values rebuilt from a cached low-rank latent, a rotated key part shared by
all heads, interleaved rotary pairing, a sink per head in the softmax's denominator). The feed-forward is dense with
the PolyNorm activation, or a mixture of SiLU-gated experts (sigmoid router with a correction for the choice, groups
of experts, a shared expert), or absent. A range of layers may run several times in a row with the same weights, a
cache of its own per pass, and a vector of its own added to the stream in front of every pass. config.json gives every
size and constant."""
from __future__ import annotations

import dataclasses
import json
from collections.abc import Mapping
from typing import Any

from ..config.model import ConfigError, eos_ids
from ..config.model import config_value as _get
from ..registry import register_architecture
from ..spec import LayerSpec, ModelSpec, PartRef, WeightRule, looped_order

NAME = "Nevodra"
MIXERS = ("attention", "latent_attention")


def _check_mlp(at: str, mlp: Mapping[str, Any]) -> None:
    kind = _get(mlp, "kind")
    if kind == "dense":
        _get(mlp, "ff", int)
    elif kind == "moe":
        _get(mlp, "expert.ff", int)
        experts, top = _get(mlp, "router.experts", int), _get(mlp, "router.top", int)
        _get(mlp, "router.scale", float)
        if top > experts:
            raise ConfigError(f"{at}: router.top {top} exceeds router.experts {experts}")
        groups = mlp["router"].get("groups")
        if groups:
            count, keep = _get(groups, "count", int), _get(groups, "keep", int)
            if experts % count or keep > count or top > keep * (experts // count):
                raise ConfigError(f"{at}: {experts} experts do not form {count} equal groups of which {keep} can hold "
                                  f"the {top} chosen")
        if mlp.get("shared"):
            _get(mlp, "shared.ff", int)
    else:
        raise ConfigError(f"{at}: unknown feed-forward kind {kind!r} (dense, moe)")


@dataclasses.dataclass(frozen=True)
class NevodraConfig:
    width: int
    vocab: int
    eps: float
    embedding_scale: float
    layers: tuple                                 # per layer: its config.json entry (type, mixer, mlp), checked
    canon_taps: int = 0                           # 0: no filter on the sublayers' inputs
    loop: tuple[int, int, int] | None = None      # (start, stop, times)
    eos_token_ids: tuple[int, ...] = ()
    architecture: str = NAME

    @classmethod
    def from_dict(cls, c: Mapping[str, Any], generation: Mapping[str, Any] | None = None) -> "NevodraConfig":
        width, vocab = _get(c, "width", int), _get(c, "vocab", int)
        eps = _get(c, "norm.eps", float)
        scale = _get(c, "embedding.scale", float) if c.get("embedding") else 1.0
        layers = _get(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("`layers` must be a non-empty list")
        for i, layer in enumerate(layers):
            at = f"layers[{i}]"
            kind, m = _get(layer, "type"), _get(layer, "mixer")
            if kind == "attention":
                for key in ("heads", "dim", "vdim"):
                    _get(m, key, int)
                _get(m, "scale", float)
                if m.get("kv_heads") is not None:
                    _get(m, "kv_heads", int)
                    if m["heads"] % m["kv_heads"]:
                        raise ConfigError(f"{at}: heads {m['heads']} are not a multiple of kv_heads {m['kv_heads']}")
                if m.get("mask"):
                    _get(m, "mask.size", int)
                    keep = m["mask"].get("keep_first", 0)
                    if not isinstance(keep, int) or isinstance(keep, bool) or keep < 0:
                        raise ConfigError(f"{at}: mask.keep_first must be a count of tokens, got {keep!r}")
                if m.get("softcap") is not None and not _get(m, "softcap", float) > 0:
                    raise ConfigError(f"{at}: softcap must be positive")
            elif kind == "latent_attention":
                for key in ("heads", "dim", "vdim", "kv_rank"):
                    _get(m, key, int)
                _get(m, "scale", float)
                rot_dim = m.get("rot_dim", 0)
                if not isinstance(rot_dim, int) or isinstance(rot_dim, bool) or rot_dim < 0:
                    raise ConfigError(f"{at}: rot_dim must be a count of dimensions, got {rot_dim!r}")
                if rot_dim:
                    dims = _get(m, "rot.dims", int)
                    _get(m, "rot.base", float)
                    if dims % 2 or dims > rot_dim:
                        raise ConfigError(f"{at}: rot.dims {dims} must be even and within rot_dim {rot_dim}")
            else:
                raise ConfigError(f"{at}: unknown layer type {kind!r} ({', '.join(MIXERS)})")
            if layer.get("mlp"):
                _check_mlp(at, layer["mlp"])
        loop = c.get("loop") or None
        if loop:
            start, stop, times = (_get(loop, key) for key in ("start", "stop", "times"))
            if not (all(isinstance(v, int) and not isinstance(v, bool) for v in (start, stop, times))
                    and 0 <= start < stop <= len(layers) and times >= 1):
                raise ConfigError(f"loop {dict(loop)} must name layers start < stop within the model and times >= 1")
            loop = (start, stop, times)
        taps = _get(c, "canon.taps", int) if c.get("canon") else 0
        return cls(width=width, vocab=vocab, eps=eps, embedding_scale=scale, layers=tuple(json.loads(json.dumps(layers))),
                   canon_taps=taps, loop=loop, eos_token_ids=eos_ids(c, generation))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
                               "norm": {"eps": self.eps}, "embedding": {"scale": self.embedding_scale},
                               "layers": list(self.layers)}
        if self.canon_taps:
            out["canon"] = {"taps": self.canon_taps}
        if self.loop:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out


def _rules(loop_start: int | None) -> tuple[WeightRule, ...]:
    mix, ffn = "layers.{i}.mixer.", "layers.{i}.ffn."
    rules = [WeightRule("embed", "embed.weight"), WeightRule("head", "lm_head.weight"),
             WeightRule("final.norm", "norm.weight"),
             WeightRule("l{i}.norm1", "layers.{i}.norm1.weight"), WeightRule("l{i}.norm2", "layers.{i}.norm2.weight"),
             WeightRule("l{i}.canon1", "layers.{i}.conv1.weight"), WeightRule("l{i}.canon2", "layers.{i}.conv2.weight")]
    if loop_start is not None:
        rules.append(WeightRule("loop.step", f"layers.{loop_start}.step"))
    # the two mixers (q and o are shared names)
    rules += [WeightRule(f"l{{i}}.mix.{s}.norm", f"{mix}{s}_norm") for s in ("q", "k")]
    rules += [WeightRule("l{i}.mix.dkv.norm", f"{mix}dkv_norm.weight")]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}.weight") for s in ("q", "k", "v", "o", "dkv")]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}") for s in ("r1", "r2", "sink", "uk", "uv")]
    # the feed-forwards
    rules += [WeightRule(f"l{{i}}.mlp.e{{e}}.{s}", f"{ffn}{s}", "e") for s in ("gate", "up", "down")]
    rules += [WeightRule(f"l{{i}}.mlp.shared.{s}", f"{ffn}shared_{s}") for s in ("gate", "up", "down")]
    rules += [WeightRule(f"l{{i}}.mlp.{s}", f"{ffn}{s}") for s in ("router", "correction", "act")]
    rules += [WeightRule(f"l{{i}}.mlp.{s}", f"{ffn}{s}_proj.weight") for s in ("up", "down")]
    return tuple(rules)


def _mixer(c: NevodraConfig, layer: Mapping[str, Any]) -> PartRef:
    m = layer["mixer"]
    if layer["type"] == "attention":
        mask = m.get("mask") or {}
        return PartRef("mixer", "attention", heads=m["heads"], kv_heads=m.get("kv_heads") or m["heads"], dim=m["dim"],
                       vdim=m["vdim"], scale=float(m["scale"]), whole_norm=c.eps, softcap=float(m.get("softcap") or 0.0),
                       distance_bias=True, window=mask.get("size", 0), keep_first=mask.get("keep_first", 0))
    rot_dim = m.get("rot_dim", 0)
    position = None
    if rot_dim:
        position = PartRef("position", "rope_yarn", theta=float(m["rot"]["base"]), rotary_dim=m["rot"]["dims"],
                           interleaved=True)
    return PartRef("mixer", "latent_attention", heads=m["heads"], dim=m["dim"], vdim=m["vdim"], kv_rank=m["kv_rank"],
                   rot_dim=rot_dim, position=position, sink=True, scale=float(m["scale"]),
                   norm=PartRef("norm", "rmsnorm", eps=c.eps))


def _ffn(c: NevodraConfig, mlp: Mapping[str, Any] | None) -> PartRef | None:
    if not mlp:
        return None
    if mlp["kind"] == "dense":
        return PartRef("ffn", "polynorm", inter=mlp["ff"], eps=c.eps)
    router = mlp["router"]
    groups = router.get("groups") or {}
    return PartRef("ffn", "moe", experts=router["experts"], top=router["top"], inter=mlp["expert"]["ff"],
                   scale=float(router["scale"]), groups=groups.get("count", 1), keep=groups.get("keep", 1), bias=True,
                   shared=(mlp.get("shared") or {}).get("ff", 0))


def recipe(c: NevodraConfig) -> ModelSpec:
    norm = PartRef("norm", "rms32", eps=c.eps)
    layers, skip = [], []
    for i, layer in enumerate(c.layers):
        ffn = _ffn(c, layer.get("mlp"))
        opens = bool(c.loop) and i == c.loop[0]
        block = PartRef("block", "parallel32", conv_taps=c.canon_taps, pass_steps=c.loop[2] if opens else 0)
        layers.append(LayerSpec(block=block, mixer=_mixer(c, layer), ffn=ffn, norm=norm))
        if ffn is None:                            # a layer without feed-forward may still list what would lead to it
            skip += [f"l{i}.norm2", f"l{i}.canon2"]
    return ModelSpec(hidden=c.width, vocab=c.vocab, layers=tuple(layers), order=looped_order(len(layers), c.loop),
                     embed=PartRef("embed", "table", scale=c.embedding_scale), norm=norm,
                     head=PartRef("head", "linear", tied=False), rules=_rules(c.loop[0] if c.loop else None),
                     skip=tuple(skip), eos_token_ids=c.eos_token_ids)


register_architecture(NAME, NevodraConfig, recipe)
