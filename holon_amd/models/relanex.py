"""Relanex: its typed configuration, and configuration to spec.

A decoder whose norm is the Dynamic Tanh (no statistics), with one in front of and one behind every sublayer, over a
residual stream kept in float32: x += m post(sublayer(pre(x))), m = `residual_mult`. The embedding's rows go through
the norm too. Each layer names its mixer: `attention` (grouped-query softmax attention with biases, interleaved rotary
positions on part of the head with YaRN's rescaling, and a sink per head), `latent_attention` (queries, keys and
values through low-rank latents, a sliding window, no positions; the latent alone is cached) or `mlstm` (the matrix
memory of xLSTM); a layer may have no feed-forward (SiLU-gated otherwise). A range of layers may run several times in
a row with the same weights and a cache of its own per pass; in front of every pass but the first the embedding's
output is added to the stream. config.json gives every size and constant."""
from __future__ import annotations

import dataclasses
import json
from collections.abc import Mapping
from typing import Any

from ..config.model import ConfigError, eos_ids
from ..config.model import config_value as _get
from ..registry import register_architecture
from ..spec import LayerSpec, ModelSpec, PartRef, WeightRule, looped_order

NAME = "Relanex"
MIXERS = ("attention", "latent_attention", "mlstm")


@dataclasses.dataclass(frozen=True)
class RelanexConfig:
    width: int
    vocab: int
    eps: float
    residual_mult: float
    layers: tuple                                 # per layer: its config.json entry (type, mixer, mlp), checked
    loop: tuple[int, int, int] | None = None      # (start, stop, times)
    eos_token_ids: tuple[int, ...] = ()
    architecture: str = NAME

    @classmethod
    def from_dict(cls, c: Mapping[str, Any], generation: Mapping[str, Any] | None = None) -> "RelanexConfig":
        width, vocab = _get(c, "width", int), _get(c, "vocab", int)
        eps, mult = _get(c, "norm.eps", float), _get(c, "residual_mult", float)
        layers = _get(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("`layers` must be a non-empty list")
        for i, layer in enumerate(layers):
            at = f"layers[{i}]"
            kind, m = _get(layer, "type"), _get(layer, "mixer")
            if kind == "attention":
                for key in ("heads", "kv_heads", "dim", "vdim"):
                    _get(m, key, int)
                _get(m, "scale", float)
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{at}: heads {m['heads']} are not a multiple of kv_heads {m['kv_heads']}")
                rot = m.get("rot")
                if rot:
                    _get(rot, "dims", int)
                    _get(rot, "base", float)
                    if rot["dims"] % 2 or rot["dims"] > m["dim"]:
                        raise ConfigError(f"{at}: rot.dims {rot['dims']} must be even and within dim {m['dim']}")
                    if rot.get("scaling"):
                        for key in ("factor", "original", "fast", "slow"):
                            _get(rot["scaling"], key, float)
            elif kind == "latent_attention":
                for key in ("heads", "dim", "vdim", "q_rank", "kv_rank", "mask.size"):
                    _get(m, key, int)
                _get(m, "scale", float)
            elif kind == "mlstm":
                for key in ("heads", "dim", "vdim"):
                    _get(m, key, int)
                if not _get(m, "gate_cap", float) > 0:
                    raise ConfigError(f"{at}: gate_cap must be positive")
            else:
                raise ConfigError(f"{at}: unknown layer type {kind!r} ({', '.join(MIXERS)})")
            mlp = layer.get("mlp")
            if mlp:
                if _get(mlp, "kind") != "dense":
                    raise ConfigError(f"{at}: unknown feed-forward kind {mlp['kind']!r} (dense)")
                _get(mlp, "ff", int)
        loop = c.get("loop") or None
        if loop:
            start, stop, times = (_get(loop, key) for key in ("start", "stop", "times"))
            if not (all(isinstance(v, int) and not isinstance(v, bool) for v in (start, stop, times))
                    and 0 <= start < stop <= len(layers) and times >= 1):
                raise ConfigError(f"loop {dict(loop)} must name layers start < stop within the model and times >= 1")
            loop = (start, stop, times)
        return cls(width=width, vocab=vocab, eps=eps, residual_mult=mult, layers=tuple(json.loads(json.dumps(layers))),
                   loop=loop, eos_token_ids=eos_ids(c, generation))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
                               "norm": {"eps": self.eps}, "residual_mult": self.residual_mult,
                               "layers": list(self.layers)}
        if self.loop:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out


def _norm_rules(name: str, target: str) -> list[WeightRule]:
    return [WeightRule(name, f"{target}.weight"), WeightRule(f"{name}.b", f"{target}.bias"),
            WeightRule(f"{name}.alpha", f"{target}.alpha")]


def _rules() -> tuple[WeightRule, ...]:
    mix = "layers.{i}.mixer."
    rules = [WeightRule("embed", "embed.weight"), WeightRule("head", "lm_head.weight")]
    rules += _norm_rules("embed.norm", "embed.norm") + _norm_rules("final.norm", "norm")
    for n in ("norm1", "norm1b", "norm2", "norm2b"):
        rules += _norm_rules(f"l{{i}}.{n}", f"layers.{{i}}.{n}")
    rules += [WeightRule(f"l{{i}}.mlp.{s}", f"layers.{{i}}.ffn.{s}_proj.weight") for s in ("gate", "up", "down")]
    # projections of the three mixers (q, k, v, o are shared names)
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}.weight") for s in ("q", "k", "v", "g", "o", "i", "f", "dq", "uq",
                                                                           "dkv")]
    rules += [WeightRule(f"l{{i}}.mix.{s}.b", f"{mix}{s}_bias") for s in ("q", "k", "v", "i", "f")]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}") for s in ("sink", "norm", "uk", "uv")]
    rules += [WeightRule(f"l{{i}}.mix.{s}.norm", f"{mix}{s}_norm.weight") for s in ("dq", "dkv")]
    return tuple(rules)


def recipe(c: RelanexConfig) -> ModelSpec:
    norm = PartRef("norm", "dyt", eps=c.eps)
    layers = []
    for i, layer in enumerate(c.layers):
        m = layer["mixer"]
        if layer["type"] == "attention":
            rot = m.get("rot")
            position = None
            if rot:
                scaling = tuple(sorted(rot["scaling"].items())) if rot.get("scaling") else None
                position = PartRef("position", "rope_yarn", theta=float(rot["base"]), rotary_dim=rot["dims"],
                                   scaling=scaling, interleaved=True)
            mixer = PartRef("mixer", "attention", heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"],
                            vdim=m["vdim"], scale=float(m["scale"]), qkv_bias=True, sink=True, position=position)
        elif layer["type"] == "latent_attention":
            mixer = PartRef("mixer", "latent_attention", heads=m["heads"], dim=m["dim"], vdim=m["vdim"],
                            q_rank=m["q_rank"], kv_rank=m["kv_rank"], scale=float(m["scale"]),
                            window=m["mask"]["size"], norm=PartRef("norm", "rmsnorm", eps=c.eps))
        else:
            mixer = PartRef("mixer", "mlstm", heads=m["heads"], dim=m["dim"], vdim=m["vdim"],
                            gate_cap=float(m["gate_cap"]), eps=c.eps)
        mlp = layer.get("mlp")
        ffn = PartRef("ffn", "swiglu", inter=mlp["ff"]) if mlp else None
        block = PartRef("block", "sandwich32", scale=c.residual_mult, reentry=bool(c.loop) and i == c.loop[0])
        layers.append(LayerSpec(block=block, mixer=mixer, ffn=ffn, norm=norm))
    return ModelSpec(hidden=c.width, vocab=c.vocab, layers=tuple(layers), order=looped_order(len(layers), c.loop),
                     embed=PartRef("embed", "table", norm=norm), norm=norm, head=PartRef("head", "linear", tied=False),
                     rules=_rules(), eos_token_ids=c.eos_token_ids)


register_architecture(NAME, RelanexConfig, recipe)
