"""Dopirax: its typed configuration, and configuration to spec.

A decoder whose two sublayers read one norm of the residual stream, x += mixer(a) + ffn(a) with a = norm(x), the
stream kept in float32 and the norm an RMS norm whose weight is kept as an offset w from one (it multiplies by 1 + w). The
embedding's rows are multiplied by a constant. Each layer names its mixer: `attention` (grouped-query softmax
attention with biases on the query, key and output projections, no value projection (a token's values are its keys
before the rotation), rotary positions on the first dimensions of a head in the half-split pairing, scores squashed by
a tanh cap, a softmax whose denominator holds one more term, exp(0), and one sigmoid gate a head on the result) or `attention_2`
(differential attention: two softmax maps a head over one set of values, queries and keys RMS-normed per head and map
and turned in the interleaved pairing, the second map's result taken off the first's with a factor the layer learns,
the difference divided by its root mean square; such a layer may have no keys and values of its own and read those an
earlier layer cached). The feed-forward is dense with a squared ReLU, or a mixture of SiLU-gated experts (logits with
a bias, the largest chosen, weights the softmax over the chosen ones; a shared expert behind a sigmoid gate a token),
or absent. config.json gives every size and constant."""
from __future__ import annotations

import dataclasses
import json
from collections.abc import Mapping
from typing import Any

from ..config.model import ConfigError, eos_ids
from ..config.model import config_value as _get
from ..registry import register_architecture
from ..spec import LayerSpec, ModelSpec, PartRef, Run, WeightRule

NAME = "Dopirax"
MIXERS = ("attention", "attention_2")


def _check_mlp(at: str, mlp: Mapping[str, Any]) -> None:
    kind = _get(mlp, "kind")
    if kind == "dense":
        _get(mlp, "ff", int)
    elif kind == "moe":
        _get(mlp, "expert.ff", int)
        experts, top = _get(mlp, "router.experts", int), _get(mlp, "router.top", int)
        if top > experts:
            raise ConfigError(f"{at}: router.top {top} exceeds router.experts {experts}")
        if mlp.get("shared"):
            _get(mlp, "shared.ff", int)
    else:
        raise ConfigError(f"{at}: unknown feed-forward kind {kind!r} (dense, moe)")


def _check_rot(at: str, m: Mapping[str, Any]) -> None:
    if m.get("rot"):
        dims = _get(m, "rot.dims", int)
        _get(m, "rot.base", float)
        if dims % 2 or dims > m["dim"]:
            raise ConfigError(f"{at}: rot.dims {dims} must be even and within dim {m['dim']}")


@dataclasses.dataclass(frozen=True)
class DopiraxConfig:
    width: int
    vocab: int
    eps: float
    embedding_scale: float
    layers: tuple                                 # per layer: its config.json entry (type, mixer, mlp), checked
    eos_token_ids: tuple[int, ...] = ()
    architecture: str = NAME

    @classmethod
    def from_dict(cls, c: Mapping[str, Any], generation: Mapping[str, Any] | None = None) -> "DopiraxConfig":
        width, vocab = _get(c, "width", int), _get(c, "vocab", int)
        eps = _get(c, "norm.eps", float)
        scale = _get(c, "embedding.scale", float) if c.get("embedding") else 1.0
        layers = _get(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("`layers` must be a non-empty list")
        layers = json.loads(json.dumps(layers))            # a copy: defaults are filled in below
        for i, layer in enumerate(layers):
            at = f"layers[{i}]"
            kind, m = _get(layer, "type"), _get(layer, "mixer")
            if kind not in MIXERS:
                raise ConfigError(f"{at}: unknown layer type {kind!r} ({', '.join(MIXERS)})")
            if not isinstance(m, Mapping):
                raise ConfigError(f"{at}: `mixer` must hold the mixer's sizes")
            if kind == "attention" and "dim" in m:
                m.setdefault("vdim", m["dim"])             # the values are the keys
            if "heads" in m:
                m.setdefault("kv_heads", m["heads"])       # no grouping named: every head has its own keys
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _get(m, key, int)
            _get(m, "scale", float)
            if m["heads"] % m["kv_heads"]:
                raise ConfigError(f"{at}: heads {m['heads']} are not a multiple of kv_heads {m['kv_heads']}")
            _check_rot(at, m)
            if kind == "attention":
                if m["vdim"] != m["dim"]:
                    raise ConfigError(f"{at}: the values are the keys, so vdim {m['vdim']} must equal dim {m['dim']}")
                if m.get("softcap") is not None and not _get(m, "softcap", float) > 0:
                    raise ConfigError(f"{at}: softcap must be positive")
            else:
                _get(m, "diff", float)
                src = m.get("kv_from")
                if src is not None:
                    if not isinstance(src, int) or isinstance(src, bool) or not 0 <= src < i:
                        raise ConfigError(f"{at}: kv_from {src!r} must name an earlier layer")
                    other = layers[src]
                    if other.get("type") != kind or other["mixer"].get("kv_from") is not None:
                        raise ConfigError(f"{at}: kv_from {src} must name an {kind} layer with keys and values of its own")
                    same = ("kv_heads", "dim", "vdim", "rot")
                    if any(other["mixer"].get(key) != m.get(key) for key in same):
                        raise ConfigError(f"{at}: layer {src}'s kv_heads, dim, vdim and rot must equal this layer's")
            if layer.get("mlp"):
                _check_mlp(at, layer["mlp"])
        return cls(width=width, vocab=vocab, eps=eps, embedding_scale=scale, layers=tuple(layers),
                   eos_token_ids=eos_ids(c, generation))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
                               "norm": {"eps": self.eps}, "embedding": {"scale": self.embedding_scale},
                               "layers": list(self.layers)}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out


def _rules() -> tuple[WeightRule, ...]:
    mix, ffn = "layers.{i}.mixer.", "layers.{i}.ffn."
    rules = [WeightRule("embed", "embed.weight"), WeightRule("head", "lm_head.weight"),
             WeightRule("final.norm", "norm.weight"), WeightRule("l{i}.norm1", "layers.{i}.norm1.weight")]
    # the mixers (q, k and o are shared names); the longer names first: `{i}` alone matches digits
    rules += [WeightRule(f"l{{i}}.mix.{s}.b", f"{mix}{s}_bias") for s in ("q", "k", "o")]
    rules += [WeightRule(f"l{{i}}.mix.{s}.norm", f"{mix}{s}_norm") for s in ("q", "k")]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}.weight") for s in ("q", "k", "v", "g", "o")]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}") for s in ("lq1", "lk1", "lq2", "lk2")]
    # the feed-forwards
    rules += [WeightRule(f"l{{i}}.mlp.e{{e}}.{s}", f"{ffn}{s}", "e") for s in ("gate", "up", "down")]
    rules += [WeightRule(f"l{{i}}.mlp.shared.{s}", f"{ffn}shared_{s}") for s in ("gate", "up", "down", "sg")]
    rules += [WeightRule("l{i}.mlp.router.b", f"{ffn}router_bias"), WeightRule("l{i}.mlp.router", f"{ffn}router")]
    rules += [WeightRule(f"l{{i}}.mlp.{s}", f"{ffn}{s}_proj.weight") for s in ("up", "down")]
    return tuple(rules)


def _position(m: Mapping[str, Any], interleaved: bool) -> PartRef | None:
    if not m.get("rot"):
        return None
    return PartRef("position", "rope_yarn", theta=float(m["rot"]["base"]), rotary_dim=m["rot"]["dims"],
                   interleaved=interleaved)


def _mixer(c: DopiraxConfig, layer: Mapping[str, Any]) -> PartRef:
    m = layer["mixer"]
    if layer["type"] == "attention":
        return PartRef("mixer", "attention", heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"],
                       scale=float(m["scale"]), softcap=float(m.get("softcap") or 0.0), qkv_bias=True, o_bias=True,
                       values_from_keys=True, sink_value=0.0, head_gate=True, position=_position(m, False))
    return PartRef("mixer", "diff_attention", heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"],
                   scale=float(m["scale"]), diff=float(m["diff"]), eps=c.eps, position=_position(m, True),
                   own_kv=m.get("kv_from") is None)


def _ffn(mlp: Mapping[str, Any] | None) -> PartRef | None:
    if not mlp:
        return None
    if mlp["kind"] == "dense":
        return PartRef("ffn", "dense", inter=mlp["ff"], act="relu2")
    shared = (mlp.get("shared") or {}).get("ff", 0)
    return PartRef("ffn", "moe", experts=mlp["router"]["experts"], top=mlp["router"]["top"], inter=mlp["expert"]["ff"],
                   score="softmax_top", bias=True, shared=shared, shared_gated=bool(shared))


def recipe(c: DopiraxConfig) -> ModelSpec:
    norm = PartRef("norm", "rms32", eps=c.eps, one_plus=True)
    block = PartRef("block", "parallel32", shared_norm=True)
    layers = tuple(LayerSpec(block=block, mixer=_mixer(c, layer), ffn=_ffn(layer.get("mlp")), norm=norm)
                   for layer in c.layers)
    # every layer runs once, so a run's place in the order is its layer's number
    order = tuple(Run(i, reads=layer["mixer"].get("kv_from")) for i, layer in enumerate(c.layers))
    return ModelSpec(hidden=c.width, vocab=c.vocab, layers=layers, order=order,
                     embed=PartRef("embed", "table", scale=c.embedding_scale), norm=norm,
                     head=PartRef("head", "linear", tied=False), rules=_rules(), eos_token_ids=c.eos_token_ids)


register_architecture(NAME, DopiraxConfig, recipe)
